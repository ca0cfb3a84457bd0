// Causal grouped-query attention for long portions (prefill) on the matrix cores, with the keys
// and values of a block staged in LDS and shared by the four waves of a workgroup.
//
// The one-wave kernel (attention_mfma_impl.h) has every wave read its keys and values from the
// cache itself; for a long portion the same block is then fetched by every tile of the request,
// and the kernel is bound by those fetches (L2 to compute unit), far from the matrix cores' rate.
// Here a workgroup takes up to four consecutive tiles of one request and kv head (32 query rows
// each: tokens x heads of the group), one per wave.  All 256 threads copy a block of 64 keys and
// values from the cache pages into LDS with fully coalesced 16-byte loads (the next block's loads
// are in flight while the present one is computed: two LDS buffers, one barrier per block); every
// wave then takes its A operands from LDS.
//
// The arithmetic is that of the one-wave kernel, computed transposed so that no operand changes
// lanes:  S^T[key, row] = K . Q^T  (v_mfma_f32_16x16x32_bf16 over the head dimension),  softmax
// over the keys of a column in float32 with running maximum and sum,  O^T += V^T . P^T.
// Row c of score tile t of a group of 32 keys is key 8 (c / 4) + 4 t + c % 4: lane group G then
// holds, over the two tiles, the probabilities of keys 8 G .. 8 G + 7 in order, which is the B
// operand of one 16x16x32 product over 32 keys, with V^T[d, 8 G .. 8 G + 7] (16 bytes of LDS) as A.
//
// Requires head_dim a multiple of 32 (up to 256) and a page size of 8, 16, 32 or 64.
#include "attention_mfma_impl.h"

#include <type_traits>

// Padding of the rows of K and of V^T in LDS, in elements (multiples of 8: rows stay 16-byte
// aligned).  Measured on MI355X at 28/4 heads of 128 and 2,048 tokens: without padding 91 us (K) and
// 77 us (V) against 70 us with 8; 16, 24 or 40 change nothing (178 to 184 us at 4,096 tokens for all
// of them): with 8 the layout is free of the conflicts that cost time, and what the counter of
// bank conflicts still shows does not bound the kernel.
// 1: the second batch of a die's workgroups takes its groups in ascending length (see the kernel)
#ifndef FSIE_LDS_PAIR
#define FSIE_LDS_PAIR 1
#endif
#ifndef FSIE_LDS_KPAD
#define FSIE_LDS_KPAD 8
#endif
#ifndef FSIE_LDS_VPAD
#define FSIE_LDS_VPAD 8
#endif

namespace fsie_attn {

constexpr int kLdsKeys = 64;   // keys per block
constexpr int kLdsWaves = 4;   // waves = tiles per workgroup
constexpr int kLdsThreads = 64 * kLdsWaves;

// Whether, with a page size known at compile time, all 256 threads copy from one page in each of
// their steps: step i of K and step i of V then both read page i of the block.
template <int HDT, int PS>
constexpr bool one_page_per_step() {
    if (PS <= 0) return false;
    for (int i = 0; i < HDT / 2; ++i)
        for (int t = 0; t < kLdsThreads; ++t) {
            const int p = t + kLdsThreads * i;
            if ((p / (2 * HDT)) / PS != i || (p / (PS / 8)) / (HDT * 16) != i) return false;
        }
    return true;
}

// PS: the page size where it is known when the kernel is compiled (16, the engine's default), 0 = the
// run-time argument.  With a known page size the pieces a thread copies for one step i all lie in
// one page, the same for the whole workgroup: the table entries come through the scalar unit and
// the loads take a scalar base and a per-thread offset that never changes.
template <int HDT, int PS>
__global__ __launch_bounds__(kLdsThreads) __attribute__((amdgpu_waves_per_eu(HDT <= 8 ? 2 : 1, HDT <= 8 ? 2 : 1))) void attention_mfma_lds_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_pages,
    const int32_t* __restrict__ items, const int32_t* __restrict__ groups, bf16_t* __restrict__ out, int n_heads,
    int n_kv, int page_size_arg, int window, float scale, int gh, int head_chunks, int n_groups, int n_y,
    int units_per_die) {
    constexpr int HD = HDT * 16;
    const int page_size = PS > 0 ? PS : page_size_arg;
    constexpr int S32 = HDT / 2;       // 32-wide steps over the head dimension
    constexpr int NT = 2;              // query tiles of 16 rows per wave
    constexpr int KS = HD + FSIE_LDS_KPAD;         // elements per key row in LDS (padded against bank conflicts)
    constexpr int VS = kLdsKeys + FSIE_LDS_VPAD;   // elements per dimension row of V^T in LDS
    constexpr int PER_THREAD = HDT / 2;  // 16-byte pieces of K, and of V, per thread and block
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][kLdsKeys * KS];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][HD * VS];

    // the groups are listed by ascending position, and a later group has more keys to read: the
    // grid takes them from the back, so that the longest workgroups start first
    // Which group and which kv head (and chunk of its heads): with a two-dimensional grid, blockIdx
    // says so.  With a one-dimensional grid (n_y = kv heads x chunks divides the 8 dies of the
    // device) consecutive workgroups go to consecutive dies, and die x takes y = x % n_y only:
    // the keys and values of a kv head are then read through one die's L2 cache (two dies for 4 kv
    // heads) and not through all eight.
    int g_lin = blockIdx.x, by = blockIdx.y;
    if (n_y > 0) {
        const int die = blockIdx.x & 7;
        by = die % n_y;
        const int per = 8 / n_y, sub = die / n_y;
        int i = blockIdx.x >> 3;  // the i-th workgroup of this die
#if FSIE_LDS_PAIR
        // A die's first `units_per_die` workgroups get a compute unit each, the next as many join
        // them there in the same order (two fit a unit), and only what follows waits for a free
        // place.  The first batch takes the longest groups in descending order; the second batch is
        // turned round, so that the unit with the longest group of the first gets the shortest of the
        // second: with 2,048 tokens (56 workgroups a die) the fullest unit then has 32 blocks of
        // keys to go through, not 46.
        if (i >= units_per_die && i < 2 * units_per_die) {
            const int n_local = (n_groups - sub + per - 1) / per;
            const int hi = min(2 * units_per_die, n_local);
            if (i < hi) i = units_per_die + (hi - 1 - i);
        }
#endif
        g_lin = i * per + sub;
        if (g_lin >= n_groups) return;
    }
    const int g_idx = n_groups - 1 - g_lin;
    const int first = groups[2 * g_idx], n_tiles = groups[2 * g_idx + 1];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const bool active = wave < n_tiles;
    const int32_t* item = items + static_cast<int64_t>(first + (active ? wave : 0)) * FSIE_ATTN_ITEM_INTS;
    // the same for every lane of the wave: kept in scalar registers, so that what is decided by
    // them is a scalar branch and not a masked region
    const int q_row0 = __builtin_amdgcn_readfirstlane(item[FSIE_ATTN_ITEM_QROW]);
    const int n_q = __builtin_amdgcn_readfirstlane(item[FSIE_ATTN_ITEM_NQ]);
    const int pos0 = __builtin_amdgcn_readfirstlane(item[FSIE_ATTN_ITEM_POS]);
    const int key_begin = __builtin_amdgcn_readfirstlane(item[FSIE_ATTN_ITEM_KBEGIN]);
    const int key_end = __builtin_amdgcn_readfirstlane(item[FSIE_ATTN_ITEM_KEND]);
    // the workgroup's keys: from the first tile's first to the last tile's last
    const int wg_begin = items[static_cast<int64_t>(first) * FSIE_ATTN_ITEM_INTS + FSIE_ATTN_ITEM_KBEGIN] & ~(kLdsKeys - 1);
    const int wg_end = items[static_cast<int64_t>(first + n_tiles - 1) * FSIE_ATTN_ITEM_INTS + FSIE_ATTN_ITEM_KEND];

    const int group = n_heads / n_kv;
    const int kvh = by / head_chunks;
    const int chunk = by - kvh * head_chunks;
    const int gh_here = min(gh, group - chunk * gh);
    const int h_base = kvh * group + chunk * gh;
    const int n_rows = n_q * gh;
    const int c = lane & 15;
    const int G = lane >> 4;
    // the tiles of a group belong to one request: its table's address is the same for every wave
    const int seq_wg = items[static_cast<int64_t>(first) * FSIE_ATTN_ITEM_INTS + FSIE_ATTN_ITEM_SEQ];
    const int32_t* table = block_tables + static_cast<int64_t>(seq_wg) * max_pages;
    const float scale2 = scale * kLog2e;

    // ---- this wave's queries (B operands)
    bool rvalid[NT];
    int rpos[NT], rtok[NT], rhead[NT];
    F16B qf[NT][S32];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int rg = nt * 16 + c;
        const int tq = rg / gh, hh = rg - tq * gh;
        rvalid[nt] = active && rg < n_rows && hh < gh_here;
        rtok[nt] = tq;
        rhead[nt] = h_base + hh;
        rpos[nt] = pos0 + tq;
        const bf16_t* qp = q + static_cast<int64_t>(q_row0 + (rvalid[nt] ? tq : 0)) * q_stride +
                           static_cast<int64_t>(rvalid[nt] ? rhead[nt] : h_base) * HD;
#pragma unroll
        for (int s = 0; s < S32; ++s) qf[nt][s].raw = ld16(qp + s * 32 + 8 * G);
    }
    // the running sums of the probabilities come from the matrix cores too: a row of ones beside
    // the values, so that every lane holds its row's whole sum (32 additions a block less for the
    // vector unit, which is as busy as the matrix cores here; 1 to 2 % at long portions)
    float m_run[NT];
    floatx4 l_acc[NT];
    F16B ones;
    ones.raw = uint4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    floatx4 acc[NT][HDT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m_run[nt] = -INFINITY;
        l_acc[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) acc[nt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- copying a block: thread t moves PER_THREAD pieces of K and of V
    // K: a key's row is 2 HDT pieces of 16 bytes; piece p = t + 256 i is part p % (2 HDT) of key p / (2 HDT).
    // V: the values of a page lie as [head_dim][slot]; piece p is, in memory order, piece p % cpp of
    //    dimension (p / cpp) % HD of the block's page p / (cpp HD), cpp = page_size / 8.
    // The page size is a power of two (8 to 64) that divides the block of 64 keys, and a block
    // starts at a multiple of 64: a piece's place inside its page and its page's distance from the
    // block's first page never change, so everything but the page number is computed once, here
    // (a division by a size known only at run time costs some thirty vector instructions, and
    // there were a dozen of them per thread and block).
    const int page_shift = __ffs(page_size) - 1;
    const int head_stride = page_size * HD;                 // one kv head of one page
    const uint32_t page_stride = head_stride * n_kv;        // at most 64 * 256 * kv heads elements
    const int cpp = page_size >> 3;
    const int t = threadIdx.x;
    uint4 kreg[PER_THREAD], vreg[PER_THREAD];
    int k_dst[PER_THREAD], v_dst[PER_THREAD];
    int k_key[PER_THREAD], k_pg[PER_THREAD], v_pg[PER_THREAD];
    int k_in_page[PER_THREAD], v_in_page[PER_THREAD];
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
        const int p = t + kLdsThreads * i;
        k_key[i] = p / (2 * HDT);
        const int k_part = p - k_key[i] * (2 * HDT);
        // in LDS the keys of a group of 32 lie in the order the lanes read them: key
        // 8 a + 4 tile + b (b < 4) of the group at row 16 tile + 4 a + b, so that the 16 lanes of a
        // score tile read 16 consecutive rows (no bank conflicts with the padded row length)
        const int k5 = k_key[i] & 31;
        const int row = (k_key[i] & 32) + ((k5 >> 2) & 1) * 16 + ((k5 >> 3) << 2) + (k5 & 3);
        k_dst[i] = row * KS + k_part * 8;
        k_pg[i] = k_key[i] >> page_shift;
        k_in_page[i] = kvh * head_stride + (k_key[i] & (page_size - 1)) * HD + k_part * 8;
        const int w = p % cpp, rest = p / cpp;
        const int d = rest % HD, pg = rest / HD;
        v_pg[i] = pg;
        v_in_page[i] = kvh * head_stride + d * page_size + w * 8;
        v_dst[i] = d * VS + (pg * cpp + w) * 8;  // key chunk pg * cpp + w of the block
    }
    auto fetch = [&](int kb) {
        // pages: a key without a page (past the end, or behind a window) reads page 0: finite values,
        // probability zero.  Keys past the end inside an existing page are read as they are (the
        // scores of such keys are replaced, not multiplied, and the pools hold finite values only).
        const int kb_page = kb >> page_shift;
        if constexpr (one_page_per_step<HDT, PS>()) {
            int page[PER_THREAD];
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) page[i] = table[min(kb_page + i, max_pages - 1)];
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) {
                const bool ok = kb_page + i < max_pages && page[i] >= 0;
                const uint64_t at = static_cast<uint64_t>(ok ? page[i] : 0) * page_stride;
                kreg[i] = ld16(k_pool + at + static_cast<uint32_t>(k_in_page[i]));
                vreg[i] = ld16(v_pool + at + static_cast<uint32_t>(v_in_page[i]));
            }
            return;
        }
        int kpage[PER_THREAD], vpage[PER_THREAD];
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            kpage[i] = table[min(kb_page + k_pg[i], max_pages - 1)];
            vpage[i] = table[min(kb_page + v_pg[i], max_pages - 1)];
        }
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const bool kok = kb_page + k_pg[i] < max_pages && kpage[i] >= 0;
            kreg[i] = ld16(k_pool + static_cast<uint64_t>(kok ? kpage[i] : 0) * page_stride + k_in_page[i]);
            const bool vok = kb_page + v_pg[i] < max_pages && vpage[i] >= 0;
            vreg[i] = ld16(v_pool + static_cast<uint64_t>(vok ? vpage[i] : 0) * page_stride + v_in_page[i]);
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            *reinterpret_cast<uint4*>(&k_lds[buf][k_dst[i]]) = kreg[i];
            *reinterpret_cast<uint4*>(&v_lds[buf][v_dst[i]]) = vreg[i];
        }
    };

    // ---- 32 keys of a block against this wave's rows
    const int my_last = pos0 + n_q - 1;  // no key after this position is visible to this wave

    // ---- a block of 64 keys (two halves of 32) against this wave's rows.  All scores first, so
    // that one maximum per query row serves the whole block and its two lane swaps are not waited
    // for twice; the scores stay in the units of the products and the softmax scale goes into the
    // exponent: p = exp2((s - m) * scale2), one fused multiply-add per score.
    // INNER: a block that every row of the wave sees whole (below the diagonal, inside the key range
    // and the window; in a long portion nearly every block): no masks and no branches, one
    // straight run of instructions in which the compiler can place the LDS reads of a product
    // ahead of the arithmetic that precedes it.
    auto compute_block = [&](int kb, const bf16_t* kbuf, const bf16_t* vbuf, auto inner) {
        constexpr bool INNER = decltype(inner)::value;
        bool use[2];
        floatx4 st[2][NT][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kh = kb + 32 * h;
            use[h] = INNER || (kh <= my_last && kh < key_end && kh + 32 > key_begin);  // the same for the whole wave
            if (!use[h]) continue;
            F16B kf[2][S32];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const bf16_t* kr = kbuf + (32 * h + 16 * tt + c) * KS + 8 * G;  // the row of key 8 (c / 4) + 4 tt + c % 4
#pragma unroll
                for (int s = 0; s < S32; ++s) kf[tt][s].raw = *reinterpret_cast<const uint4*>(kr + s * 32);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    floatx4 a = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < S32; ++s)
                        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tt][s].v, qf[nt][s].v, a, 0, 0, 0);
                    st[h][nt][tt] = a;
                }
        }
        // mask and maximum
        float sv[2][NT][8];
        float m_loc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) m_loc[nt] = -INFINITY;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (!use[h]) continue;
            const int kh = kb + 32 * h;
            const bool full = INNER || (kh >= key_begin && kh + 32 <= key_end && kh + 31 <= pos0 &&
                                        (window <= 0 || kh > pos0 + n_q - 1 - window));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (full) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) sv[h][nt][i] = st[h][nt][i >> 2][i & 3];
                } else {
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int key = kh + 8 * G + 4 * tt + r;
                            const bool vis = rvalid[nt] && key >= key_begin && key < key_end && key <= rpos[nt] &&
                                             (window <= 0 || key > rpos[nt] - window);
                            sv[h][nt][tt * 4 + r] = vis ? st[h][nt][tt][r] : -INFINITY;
                        }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) m_loc[nt] = fmaxf(m_loc[nt], sv[h][nt][i]);
            }
        }
        // new maxima; the accumulators shrink only when some row's maximum moved (rare after the
        // first blocks), for both tiles behind one branch, so that what follows it (the exponentials,
        // the LDS reads of the values and the second product) is one run of instructions
        float corr[NT], shift[NT];
        bool moved = false;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // the maximum never goes below a finite floor, so that a row that has seen no key yet
            // gives exp2(-inf) = 0 and not exp2(-inf + inf)
            const float m_new = fmaxf(fmaxf(m_run[nt], max_xor32(max_xor16(m_loc[nt]))), -1e30f);
            corr[nt] = __builtin_amdgcn_exp2f((m_run[nt] - m_new) * scale2);
            shift[nt] = -m_new * scale2;
            m_run[nt] = m_new;
            moved = moved || corr[nt] != 1.f;
        }
        if (__any(moved)) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                l_acc[nt][0] *= corr[nt];
                l_acc[nt][1] *= corr[nt];
                l_acc[nt][2] *= corr[nt];
                l_acc[nt][3] *= corr[nt];
#pragma unroll
                for (int dt = 0; dt < HDT; ++dt) {
                    acc[nt][dt][0] *= corr[nt];
                    acc[nt][dt][1] *= corr[nt];
                    acc[nt][dt][2] *= corr[nt];
                    acc[nt][dt][3] *= corr[nt];
                }
            }
        }
        // probabilities
        F16B pb[2][NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (!use[h]) continue;
                float p[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_exp2f(fmaf(sv[h][nt][i], scale2, shift[nt]));
                pb[h][nt].raw = uint4{pack2_bf16(p[0], p[1]), pack2_bf16(p[2], p[3]), pack2_bf16(p[4], p[5]),
                                      pack2_bf16(p[6], p[7])};
            }
        }
        // O^T += V^T P^T
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (!use[h]) continue;
            F16B vf[HDT];
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt)
                vf[dt].raw = *reinterpret_cast<const uint4*>(vbuf + (dt * 16 + c) * VS + 32 * h + 8 * G);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                l_acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pb[h][nt].v, l_acc[nt], 0, 0, 0);
#pragma unroll
                for (int dt = 0; dt < HDT; ++dt)
                    acc[nt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pb[h][nt].v, acc[nt][dt], 0, 0, 0);
            }
        }
    };

    // ---- the blocks: fetch the next one, compute the present one, put the next one into LDS
    if (wg_begin < wg_end) {
        fetch(wg_begin);
        stash(0);
        __syncthreads();
        int buf = 0;
        for (int kb = wg_begin; kb < wg_end; kb += kLdsKeys) {
            const bool more = kb + kLdsKeys < wg_end;
            if (more) fetch(kb + kLdsKeys);
            const bool inner = active && kb >= key_begin && kb + kLdsKeys <= key_end && kb + kLdsKeys - 1 <= pos0 &&
                               (window <= 0 || kb > my_last - window);
            if (inner) compute_block(kb, k_lds[buf], v_lds[buf], std::true_type{});
            else if (active) compute_block(kb, k_lds[buf], v_lds[buf], std::false_type{});
            if (more) stash(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }

    // ---- results: lane holds O^T[d = 16 dt + 4 G + r][row c]
    if (!active) return;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const float l_tot = l_acc[nt][0];
        if (!rvalid[nt]) continue;
        const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        bf16_t* o = out + (static_cast<int64_t>(q_row0 + rtok[nt]) * n_heads + rhead[nt]) * HD + 4 * G;
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) {
            uint2 w;
            w.x = pack2_bf16(acc[nt][dt][0] * inv, acc[nt][dt][1] * inv);
            w.y = pack2_bf16(acc[nt][dt][2] * inv, acc[nt][dt][3] * inv);
            *reinterpret_cast<uint2*>(o + dt * 16) = w;
        }
    }
}

template <int HDT, int PS>
int launch_lds(const bf16_t* q, int64_t q_stride, const bf16_t* k_pool, const bf16_t* v_pool,
               const int32_t* block_tables, int max_pages, const int32_t* items, const int32_t* groups, int n_groups,
               bf16_t* out, int n_heads, int n_kv, int page_size, int window, float scale, hipStream_t stream) {
    const int group = n_heads / n_kv;
    const int gh = group < 32 ? group : 32;
    const int head_chunks = (group + gh - 1) / gh;
    const int ys = n_kv * head_chunks;
    const bool by_die = ys <= 8 && 8 % ys == 0;
    // by die: every die gets the same number of workgroups, the last ones of which may be empty
    const dim3 grid = by_die ? dim3(static_cast<unsigned>((n_groups + 8 / ys - 1) / (8 / ys)) * 8) : dim3(n_groups, ys);
    attention_mfma_lds_kernel<HDT, PS><<<grid, kLdsThreads, 0, stream>>>(q, q_stride, k_pool, v_pool, block_tables, max_pages,
                                                                     items, groups, out, n_heads, n_kv, page_size,
                                                                     window, scale, gh, head_chunks, n_groups,
                                                                     by_die ? ys : 0, max(1, fsie_compute_units() / 8));
    FSIE_CHECK_LAUNCH("attention_mfma_lds");
    return 0;
}

}  // namespace fsie_attn

// 1 if the LDS-shared kernel takes this geometry.
extern "C" int fsie_attention_mfma_lds_ok(int head_dim, int page_size) {
    const bool hd_ok = head_dim > 0 && head_dim % 32 == 0 && head_dim <= 256;
    const bool page_ok = page_size == 8 || page_size == 16 || page_size == 32 || page_size == 64;
    return hd_ok && page_ok ? 1 : 0;
}

// Large items (the `large` geometry of fsie_attention_mfma: up to 32 rows each) in groups of up to
// four consecutive tiles of one request: groups[2 g] = index of the group's first item in `items`,
// groups[2 g + 1] = its number of tiles (1..4).  The tiles of a group must follow one another in
// the request (ascending positions).
extern "C" int fsie_attention_mfma_lds(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                                       const int32_t* block_tables, int max_pages, const int32_t* items,
                                       const int32_t* groups, int n_groups, void* out, int n_heads, int n_kv,
                                       int head_dim, int page_size, int window, float scale, hipStream_t stream) {
    FSIE_REQUIRE(n_groups >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0,
                 "attention_mfma_lds: heads %d must be a positive multiple of kv heads %d", n_heads, n_kv);
    FSIE_REQUIRE(fsie_attention_mfma_lds_ok(head_dim, page_size),
                 "attention_mfma_lds: head_dim %d must be a multiple of 32 up to 256 and page_size %d one of 8, 16, 32, 64",
                 head_dim, page_size);
    FSIE_REQUIRE(max_pages > 0, "attention_mfma_lds: empty block table");
    FSIE_REQUIRE(q_stride % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0,
                 "attention_mfma_lds: query rows must be 16-byte aligned");
    if (n_groups == 0) return 0;
    const bf16_t* qq = static_cast<const bf16_t*>(q);
    const bf16_t* kk = static_cast<const bf16_t*>(k_pool);
    const bf16_t* vv = static_cast<const bf16_t*>(v_pool);
    bf16_t* oo = static_cast<bf16_t*>(out);
#define FSIE_LDS_CASE(H)                                                                                           \
    case H:                                                                                                        \
        return page_size == 16                                                                                     \
                   ? fsie_attn::launch_lds<H, 16>(qq, q_stride, kk, vv, block_tables, max_pages, items, groups,    \
                                                  n_groups, oo, n_heads, n_kv, page_size, window, scale, stream)   \
                   : fsie_attn::launch_lds<H, 0>(qq, q_stride, kk, vv, block_tables, max_pages, items, groups,     \
                                                 n_groups, oo, n_heads, n_kv, page_size, window, scale, stream)
    switch (head_dim / 16) {
        FSIE_LDS_CASE(2);
        FSIE_LDS_CASE(4);
        FSIE_LDS_CASE(6);
        FSIE_LDS_CASE(8);
        FSIE_LDS_CASE(10);
        FSIE_LDS_CASE(12);
        FSIE_LDS_CASE(14);
        FSIE_LDS_CASE(16);
        default: break;
    }
#undef FSIE_LDS_CASE
    fsie_set_error("attention_mfma_lds: no kernel for head_dim %d", head_dim);
    return 1;
}
