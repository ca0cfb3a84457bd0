// Causal grouped-query attention over the pages of the cache on the matrix cores (bfloat16).
//
// One wave per work item and kv head (chunk).  Everything is computed transposed so that no
// operand ever has to change lanes or pass through LDS:
//
//   S^T[key, row] = K[key, :] . Q[row, :]      A = K rows from the cache (16 B per lane),
//                                              B = Q rows, kept in registers for the whole item
//   softmax over the keys of a column: 8 keys per lane, the rest by two lane swaps (16, 32)
//   O^T[d, row]  += V^T[d, key] . P^T[key, row] A = V^T from the cache, which stores values
//                                              transposed ([head_dim][slot]: 8 consecutive keys of
//                                              one dimension are one 16-byte load),
//                                              B = P^T, which is exactly the layout in which the
//                                              first product left S^T
//
// Keys are walked in blocks of 32, scored as two tiles of 16.  Row c of tile t is key
// 8 (c / 4) + 4 t + c % 4 of the block: lane group G then holds, over the two tiles, the scores of
// the keys 8 G .. 8 G + 7 in order, which is the B operand of one v_mfma_f32_16x16x32_bf16 over
// the block's 32 keys.
//
// The running maximum and sum of a query row and its accumulators live in the same lanes
// (column = lane % 16), so the online-softmax rescale is lane-local.  Scores use
// v_mfma_f32_16x16x32_bf16 over the head dimension (16x16x16 steps when head_dim is an odd
// multiple of 16, on an accumulator of their own).
//
// HDT = head_dim / 16, NT = column tiles of 16 query rows per wave (rows = tokens x heads of the
// kv head's group).  Requires page_size % 4 == 0; with a page size that is a multiple of 8 a
// lane's 8 values of a dimension come with one load instead of two.
//
// A workgroup may have several waves (up to MAXW; 4 when NT > 1): they split the item's key range
// into contiguous runs of blocks, and their partial results are combined inside the workgroup:
// maxima and sums through LDS, then the first wave adds the others' rescaled accumulators to its
// own in the fixed order of the waves.  Decoding against a long context therefore needs neither partial
// records in memory nor a second kernel, and the result does not depend on timing.
//
// QKV: the variant for steps of one token a request takes q, k and v as the float32 partial sums
// that a product in slices of K leaves, and finishes them itself: every workgroup adds up the
// heads it needs (its queries, and its kv head's key and value), adds the bias, rotates queries
// and key, and the workgroup whose keys end with the new one scores it from registers and writes
// it and its value into the pools.  That spares the launch between the product and attention.
#pragma once

#include "common.h"
#include "api.h"

#include <math.h>

namespace fsie_attn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

union F16B {
    uint4 raw;
    bf16x8 v;
};
union F8B {
    uint2 raw;
    shortx4 v;
};

__device__ __forceinline__ uint4 ld16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
// the same as a streaming load: for data that is read once and whose whole lines one load of a wave covers
__device__ __forceinline__ uint4 ld16_once(const bf16_t* p) {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    return uint4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ uint2 ld8(const bf16_t* p) { return *reinterpret_cast<const uint2*>(p); }

// What the QKV variant reads and writes beside the kernel's other operands.
struct QkvSums {
    const float* sums;     // [n_parts][n_tokens][width], width = (n_heads + 2 n_kv) head_dim
    const float* bias;     // [width], or null
    const float* cos_sin;  // [n_tokens][head_dim / 2] pairs (cos, sin) of each token's position
    const int32_t* slots;  // [n_tokens] slot of a token's key and value in the pools (negative: nowhere)
    bf16_t* k_out;         // the pools again, to write
    bf16_t* v_out;
    int64_t part_stride;   // n_tokens * width
    int64_t pool_slots;
    int n_parts, width;
};

// Element d of a head after the rotation of the pairs (i, i + HD / 2) by the angles whose
// cosines and sines are cs[i].  One fixed sequence of roundings, whoever asks: the key that a
// step scores from registers and its copy in the cache are the same numbers.
__device__ __forceinline__ float rotated_by(float a, float b, float cosine, float sine, bool hi) {
    const float bs = __fmul_rn(b, sine);
    return __fmaf_rn(a, cosine, hi ? bs : -bs);
}
template <int HD>
__device__ __forceinline__ float rotated(const float* head, const float2* cs, int d) {
    constexpr int half = HD / 2;
    const bool hi = d >= half;
    const float2 t = cs[hi ? d - half : d];
    return rotated_by(head[d], head[hi ? d - half : d + half], t.x, t.y, hi);
}
// The same for the elements d0 .. d0 + 7 (d0 a multiple of 8), as two bfloat16 a register: 16-byte reads.
template <int HD>
__device__ __forceinline__ uint4 rotated8(const float* head, const float2* cs, int d0) {
    constexpr int half = HD / 2;
    const bool hi = d0 >= half;
    const float4* a = reinterpret_cast<const float4*>(head + d0);
    const float4* b = reinterpret_cast<const float4*>(head + (hi ? d0 - half : d0 + half));
    const float4* t = reinterpret_cast<const float4*>(cs + (hi ? d0 - half : d0));
    const float4 a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1], t0 = t[0], t1 = t[1], t2 = t[2], t3 = t[3];
    return uint4{pack2_bf16(rotated_by(a0.x, b0.x, t0.x, t0.y, hi), rotated_by(a0.y, b0.y, t0.z, t0.w, hi)),
                 pack2_bf16(rotated_by(a0.z, b0.z, t1.x, t1.y, hi), rotated_by(a0.w, b0.w, t1.z, t1.w, hi)),
                 pack2_bf16(rotated_by(a1.x, b1.x, t2.x, t2.y, hi), rotated_by(a1.y, b1.y, t2.z, t2.w, hi)),
                 pack2_bf16(rotated_by(a1.z, b1.z, t3.x, t3.y, hi), rotated_by(a1.w, b1.w, t3.z, t3.w, hi))};
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <int HDT>
constexpr int max_waves() {
    return HDT <= 4 ? 16 : (HDT <= 8 ? 8 : 4);  // registers per wave grow with the head size
}

template <int HDT, int NT, int MAXW, bool V16, bool QKV = false>
__global__ __launch_bounds__(QKV && MAXW == 1 ? 256 : 64 * MAXW) __attribute__((amdgpu_waves_per_eu(MAXW == 1 && NT > 1 ? 2 : 1))) void attention_mfma_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_pages,
    const int32_t* __restrict__ items, bf16_t* __restrict__ out, float* __restrict__ partials, int n_heads,
    int n_kv, int page_size, int window, float scale, int gh, int head_chunks, QkvSums f) {
    static_assert(!QKV || (NT == 1 && HDT % 2 == 0), "the QKV variant: one query tile, head_dim a multiple of 32");
    constexpr int HD = HDT * 16;
    // scores: 32-wide steps over the head dimension when head_dim is a multiple of 32, else
    // 16-wide steps throughout (the two shapes are never chained on one accumulator)
    constexpr bool X32 = (HDT % 2) == 0;
    constexpr int S32 = X32 ? HDT / 2 : 0;
    constexpr int S16 = X32 ? 0 : HDT;
    constexpr int S32A = S32 > 0 ? S32 : 1;
    constexpr int S16A = S16 > 0 ? S16 : 1;

    const int32_t* item = items + static_cast<int64_t>(blockIdx.x) * FSIE_ATTN_ITEM_INTS;
    const int seq = item[FSIE_ATTN_ITEM_SEQ];
    const int q_row0 = item[FSIE_ATTN_ITEM_QROW];
    const int n_q = item[FSIE_ATTN_ITEM_NQ];
    const int pos0 = item[FSIE_ATTN_ITEM_POS];
    const int key_begin = item[FSIE_ATTN_ITEM_KBEGIN];
    int key_end = item[FSIE_ATTN_ITEM_KEND];
    const int partial_base = item[FSIE_ATTN_ITEM_PARTIAL];
    if (n_q <= 0) return;  // padding item
    // QKV: the item whose keys end with the request's new one walks the cache up to it and takes
    // the new key and value from the sums
    const bool owner = QKV && pos0 >= key_begin && pos0 < key_end;
    if (owner) key_end = pos0;
    int new_slot = -1;
    if constexpr (QKV) new_slot = f.slots[q_row0];

    const int group = n_heads / n_kv;
    const int kvh = blockIdx.y / head_chunks;
    const int chunk = blockIdx.y - kvh * head_chunks;
    const int gh_here = min(gh, group - chunk * gh);
    const int h_base = kvh * group + chunk * gh;
    const int n_rows = n_q * gh;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    // (the QKV variant of one wave is launched with four: three only help to add up the sums)
    const int n_waves = QKV && MAXW == 1 ? 1 : blockDim.x >> 6;
    const int c = lane & 15;  // column of S^T and O^T (query row of a tile); row of the A tiles
    const int G = lane >> 4;  // lane group: which 4 (or 8) of the reduction indices this lane holds
    const int32_t* table = block_tables + static_cast<int64_t>(seq) * max_pages;
    const float scale2 = scale * kLog2e;  // scores in units of log2 e: exp() becomes exp2()

    // LDS: the accumulators that the waves after the first hand over at the end; before that, in
    // the QKV variant, the heads added up from the sums (up to 16 of queries, a key, a value) and
    // the cosines and sines
    constexpr int kCombine = MAXW > 1 ? (MAXW - 1) * NT * HDT * 64 : 0;
    // a head's row in LDS is four floats longer than the head, so that the 16 rows that a wave reads
    // at once, 16 bytes each, fall into different banks
    constexpr int RS = HD + 4;
    constexpr int kHeads = QKV ? (18 * RS + HD) / 4 : 0;
    constexpr int kLds = kCombine > kHeads ? kCombine : (kHeads > 0 ? kHeads : 1);
    __shared__ floatx4 s_o[kLds];
    float* s_row = reinterpret_cast<float*>(s_o);
    float2* s_cs = reinterpret_cast<float2*>(s_row + 18 * RS);
    // The heads this workgroup needs, added up over the slices, with the bias, into LDS.  In two
    // steps: first all the reads of up to eight slices, in straight-line code (a slice past the last
    // reads the last one again, a thread without a column reads column 0), so that they are under
    // way together, and with the reads of the first keys where the same wave walks keys; then the
    // additions.  A loop of one read and one addition a slice would be a trip to memory a slice.
    // The variant of one wave is launched with four: the other three add up the sums and leave
    // after the barrier, so that the first has only its keys under way.  The hardware counts 63
    // reads of a wave at most, and a wait for one of 27 reads of sums behind 64 of keys would wait
    // for most of the keys too.
    constexpr int kThreadsLeast = MAXW == 1 ? 192 : 64 * MAXW;  // threads that add up sums
    constexpr int NJ = QKV ? (18 * HD / 4 + kThreadsLeast - 1) / kThreadsLeast : 1;  // columns of four a thread
    constexpr int PC = NJ <= 3 ? 8 : 4;                                              // slices read at once
    float4 part[NJ][PC], bias_of[NJ];
    float2 angle = float2{1.f, 0.f};
    int lds_at[NJ];
    const float* col_at[NJ];
    const int sum_thread = MAXW == 1 ? static_cast<int>(threadIdx.x) - 64 : static_cast<int>(threadIdx.x);
    const int sum_threads = MAXW == 1 ? static_cast<int>(blockDim.x) - 64 : static_cast<int>(blockDim.x);
    const bool helper = QKV && MAXW == 1 && wave > 0;  // a wave that only adds up sums
    const bool sums_here = MAXW > 1 || wave > 0;
    auto issue_sums = [&]() {
        const int q_dim = n_heads * HD, kv_dim = n_kv * HD;
        const int n_cols = (gh_here + 2) * HD;
        const float* row = f.sums + static_cast<int64_t>(q_row0) * f.width;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (j * sum_threads * 4 >= n_cols) {  // (the same for the whole workgroup: no thread has such a column)
                lds_at[j] = -1;
                continue;
            }
            const int i = (sum_thread + j * sum_threads) * 4;
            const bool has = i >= 0 && i < n_cols;
            const int ic = has ? i : 0;
            const int seg = ic / HD, d = ic - seg * HD;
            lds_at[j] = has ? seg * RS + d : -1;
            const int col = seg < gh_here ? (h_base + seg) * HD + d : q_dim + (seg - gh_here) * kv_dim + kvh * HD + d;
            col_at[j] = row + col;
#pragma unroll
            for (int u = 0; u < PC; ++u)
                part[j][u] = *reinterpret_cast<const float4*>(col_at[j] + min(u, f.n_parts - 1) * f.part_stride);
            bias_of[j] = *reinterpret_cast<const float4*>(f.bias ? f.bias + col : col_at[j]);
        }
        const float2* cs = reinterpret_cast<const float2*>(f.cos_sin) + static_cast<int64_t>(q_row0) * (HD / 2);
        angle = cs[min(max(sum_thread, 0), HD / 2 - 1)];
    };
    auto finish_sums = [&]() {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (j * sum_threads * 4 >= (gh_here + 2) * HD) continue;
            float4 a{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < PC; ++u)
                if (u < f.n_parts)
                    a = float4{a.x + part[j][u].x, a.y + part[j][u].y, a.z + part[j][u].z, a.w + part[j][u].w};
            for (int s = PC; s < f.n_parts; ++s) {  // (more slices than are read at once: a trip each)
                const float4 v = *reinterpret_cast<const float4*>(col_at[j] + s * f.part_stride);
                a = float4{a.x + v.x, a.y + v.y, a.z + v.z, a.w + v.w};
            }
            if (f.bias) a = float4{a.x + bias_of[j].x, a.y + bias_of[j].y, a.z + bias_of[j].z, a.w + bias_of[j].w};
            if (lds_at[j] >= 0) *reinterpret_cast<float4*>(s_row + lds_at[j]) = a;
        }
        for (int i = max(sum_thread, 0); i < HD / 2; i += sum_threads) {
            if (i == sum_thread) s_cs[i] = angle;
            else s_cs[i] = (reinterpret_cast<const float2*>(f.cos_sin) + static_cast<int64_t>(q_row0) * (HD / 2))[i];
        }
    };

    // ---- the item's queries: B operands, kept for the whole item
    bool rvalid[NT];
    int rpos[NT], rtok[NT], rhead[NT];
    F16B qf[NT][S32A];
    F8B qt[NT][S16A];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int rg = nt * 16 + c;
        const int tq = rg / gh, hh = rg - tq * gh;
        rvalid[nt] = rg < n_rows && hh < gh_here;
        rtok[nt] = tq;
        rhead[nt] = h_base + hh;
        rpos[nt] = pos0 + tq;
        if constexpr (!QKV) {
            const bf16_t* qp = q + static_cast<int64_t>(q_row0 + (rvalid[nt] ? tq : 0)) * q_stride +
                               static_cast<int64_t>(rvalid[nt] ? rhead[nt] : h_base) * HD;
#pragma unroll
            for (int s = 0; s < S32; ++s) qf[nt][s].raw = ld16(qp + s * 32 + 8 * G);  // a row that does not exist reads
#pragma unroll
            for (int s = 0; s < S16; ++s) qt[nt][s].raw = ld8(qp + s * 16 + 4 * G);   // the item's first row: masked later
        }
    }

    float m_run[NT], l_run[NT];
    floatx4 acc[NT][HDT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m_run[nt] = -INFINITY;
        l_run[nt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) acc[nt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // QKV: the queries (one token: row c of the tile is head c of the group) from the heads in LDS
    auto build_queries = [&]() {
        const float* head = s_row + (rvalid[0] ? c : 0) * RS;
#pragma unroll
        for (int s = 0; s < S32; ++s) qf[0][s].raw = rotated8<HD>(head, s_cs, s * 32 + 8 * G);
    };

    const int64_t head_stride = static_cast<int64_t>(page_size) * HD;  // one kv head of one page
    // key / page_size as one multiplication (the host has checked that keys * page_size < 2^32): a
    // division by a size known only at run time costs some thirty vector instructions, four times
    // per block of 32 keys
    const uint32_t page_magic = 0xFFFFFFFFu / static_cast<uint32_t>(page_size) + 1u;
    // this wave's run of key blocks
    const int kb_first = key_begin & ~31;
    const int n_blocks = (key_end - kb_first + 31) >> 5;
    // an item uses one wave per 4 blocks (128 keys) of its own when it has one query tile, per 16
    // blocks (512 keys) when it has several, however many waves the launch has: how its keys are
    // split depends on the item alone
    constexpr int kBlocksPerWave = NT == 1 ? 4 : 16;
    const int n_active = min(n_waves, max(1, (n_blocks + kBlocksPerWave - 1) / kBlocksPerWave));
    const int per_wave = (n_blocks + n_active - 1) / n_active;
    // QKV: the request's new key is a run of its own, for a wave that the keys of the cache leave
    // idle if there is one (else for the first); n_runs = waves whose results are combined
    const int new_key_wave = owner && n_active < n_waves ? n_active : 0;
    const int n_runs = owner && n_active < n_waves ? n_active + 1 : n_active;
    const int kb_begin = kb_first + wave * per_wave * 32;
    const int kb_end = min(key_end, kb_begin + per_wave * 32);
    // the keys (A operand of the scores) and values (A operand of the second product) of a block
    struct Block {
        F16B kf[2][S32A];
        F8B kt[2][S16A];
        F16B vf[HDT];
    };
    // V16: the page size is a multiple of 8, so the keys 8 G .. 8 G + 7 of a block lie in one page,
    // 16-byte aligned (a template flag: a run-time branch around the loads costs a third of the speed)
    // Where the four runs of a block's keys lie: the two tiles of 16 keys of the scores (one key
    // per lane, c) and the two runs of 4 consecutive keys per lane group of the second product
    // (never across a page: page_size % 4 == 0).  A key without a page (past the end, or behind a
    // window) points at page 0: what is read there is finite and its probability is zero.
    struct Where {
        int64_t k[2], v[2];  // element offsets into the pools
    };
    struct Asked {
        int page[4], idx[4], key[4];
    };
    auto ask_pages = [&](int kb, Asked& p) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            p.key[t] = kb + 8 * (c >> 2) + 4 * t + (c & 3);
            p.key[2 + t] = kb + 8 * G + 4 * t;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // the four table reads go out together
            p.idx[i] = static_cast<int>(__umulhi(static_cast<uint32_t>(p.key[i]), page_magic));
            p.page[i] = table[min(p.idx[i], max_pages - 1)];
        }
    };
    auto place = [&](const Asked& p, Where& at) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool ok = p.key[i] < key_end && p.idx[i] < max_pages && p.page[i] >= 0;
            const int64_t head = (static_cast<int64_t>(ok ? p.page[i] : 0) * n_kv + kvh) * head_stride;
            const int off = ok ? p.key[i] - p.idx[i] * page_size : 0;
            if (i < 2) at.k[i] = head + static_cast<int64_t>(off) * HD + (X32 ? 8 : 4) * G;
            else at.v[i - 2] = head + off + static_cast<int64_t>(c) * page_size;
        }
    };
    auto locate = [&](int kb, Where& at) {
        Asked p;
        ask_pages(kb, p);
        place(p, at);
    };
    auto load_block = [&](const Where& at, Block& blk) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const bf16_t* kp = k_pool + at.k[t];
#pragma unroll
            for (int s = 0; s < S32; ++s) blk.kf[t][s].raw = ld16(kp + s * 32);
#pragma unroll
            for (int s = 0; s < S16; ++s) blk.kt[t][s].raw = ld8(kp + s * 16);
        }
        const bf16_t* v0 = v_pool + at.v[0];
        if (V16) {
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt) {
                // (streaming loads where several waves walk long runs of keys; the short items of one wave are slower with them)
                const bf16_t* vp = v0 + static_cast<int64_t>(dt * 16) * page_size;
                blk.vf[dt].raw = MAXW > 1 ? ld16_once(vp) : ld16(vp);
            }
        } else {
            const bf16_t* v1 = v_pool + at.v[1];
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt) {
                const uint2 lo = ld8(v0 + static_cast<int64_t>(dt * 16) * page_size);
                const uint2 hi = ld8(v1 + static_cast<int64_t>(dt * 16) * page_size);
                blk.vf[dt].raw = uint4{lo.x, lo.y, hi.x, hi.y};
            }
        }
    };
    auto compute_block = [&](int kb, const Block& blk) {
        const bool full = kb >= key_begin && kb + 32 <= key_end && kb + 31 <= pos0 &&
                          (window <= 0 || kb > pos0 + n_q - 1 - window);  // the same for the whole wave
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // ---- S^T for 32 keys x 16 rows
            floatx4 st[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                st[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < S32; ++s)
                    st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kf[t][s].v, qf[nt][s].v, st[t], 0, 0, 0);
#pragma unroll
                for (int s = 0; s < S16; ++s)
                    st[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(blk.kt[t][s].v, qt[nt][s].v, st[t], 0, 0, 0);
            }
            // ---- mask, running maximum.  A block that every row of the item sees whole (below
            // the diagonal, inside the key range and the window) needs no mask; in a long
            // portion that is nearly every block.
            float sv[8];
            float m_loc = -INFINITY;
            if (full) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    sv[i] = st[i >> 2][i & 3] * scale2;
                    m_loc = fmaxf(m_loc, sv[i]);
                }
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = kb + 8 * G + 4 * t + r;
                        const bool vis = rvalid[nt] && key >= key_begin && key < key_end && key <= rpos[nt] &&
                                         (window <= 0 || key > rpos[nt] - window);
                        sv[t * 4 + r] = vis ? st[t][r] * scale2 : -INFINITY;
                        m_loc = fmaxf(m_loc, sv[t * 4 + r]);
                    }
            }
            m_loc = max_xor32(max_xor16(m_loc));
            const float m_new = fmaxf(m_run[nt], m_loc);
            const float corr = (m_run[nt] == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run[nt] - m_new);
            float p[8];
            float p_sum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                p[i] = (sv[i] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sv[i] - m_new);
                p_sum += p[i];
            }
            l_run[nt] = l_run[nt] * corr + p_sum;  // this lane's keys only; lane groups are summed at the end
            m_run[nt] = m_new;
            F16B pb;  // P^T for the keys 8 G .. 8 G + 7 of the block
            pb.raw = uint4{pack2_bf16(p[0], p[1]), pack2_bf16(p[2], p[3]), pack2_bf16(p[4], p[5]), pack2_bf16(p[6], p[7])};
            // the accumulators shrink only when some row's maximum moved (rare after the first blocks)
            if (__any(corr != 1.f)) {
#pragma unroll
                for (int dt = 0; dt < HDT; ++dt) {
                    acc[nt][dt][0] *= corr;
                    acc[nt][dt][1] *= corr;
                    acc[nt][dt][2] *= corr;
                    acc[nt][dt][3] *= corr;
                }
            }
            // ---- O^T += V^T P^T
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt)
                acc[nt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.vf[dt].v, pb.v, acc[nt][dt], 0, 0, 0);
        }
    };
    // The table reads of a block go out one block ahead, so that its data reads never wait for
    // an address.  One query tile and a moderate head size leave registers for a second block:
    // its data is in flight while the matrix cores work on the present one (few waves run here,
    // so occupancy does not hide the latency).
    constexpr bool PREFETCH = NT == 1 && HDT <= 8;
    // A workgroup of one wave (items of up to 128 keys, what a step with idle compute units is cut
    // into) has all 512 registers of its SIMD: the table reads of its four blocks go out together,
    // then all their data reads, and the products follow; one trip to memory for the addresses and
    // one for the data, where fetching a block ahead costs a trip per block (8.0 -> 7.3 us a layer for
    // eight requests of 640 keys).
    constexpr bool ALL_AHEAD = PREFETCH && MAXW == 1;
    // QKV: the new key and value, from the sums: a block of their own whose first key they are (the
    // mask hides the rest), and into the pools for the steps to come.  An idle wave does it, or the
    // first one before its walk, while its first keys from the cache are under way.
    // The stores into the pools (2 bytes a dimension for the value) are not ordered against the loads of
    // other waves and workgroups that read the 16 bytes around that slot: those lanes are masked
    // (probability zero), so the result does not depend on which bytes they see, provided they are
    // finite either way.  That is the pools' invariant: a slot at or after a request's length holds a
    // finite value (a page is zeroed by the step that takes it; the null page is never written).
    auto score_new_key = [&]() {
        if (!(owner && wave == new_key_wave)) return;
        key_end = pos0 + 1;
        const float* kh = s_row + gh_here * RS;
        const float* vh = kh + RS;
        Block nb;
#pragma unroll
        for (int s = 0; s < S32; ++s) {
            const uint4 r = rotated8<HD>(kh, s_cs, s * 32 + 8 * G);
            nb.kf[0][s].raw = c == 0 ? r : uint4{0u, 0u, 0u, 0u};
            nb.kf[1][s].raw = uint4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt)
            nb.vf[dt].raw = uint4{G == 0 ? pack2_bf16(vh[dt * 16 + c], 0.f) : 0u, 0u, 0u, 0u};
        compute_block(pos0, nb);
        key_end = pos0;
        if (chunk == 0 && new_slot >= 0 && new_slot < f.pool_slots) {
            const int page = new_slot / page_size;
            const int off = new_slot - page * page_size;
            bf16_t* kd = f.k_out + ((static_cast<int64_t>(page) * n_kv + kvh) * page_size + off) * HD;
            for (int d = 2 * lane; d < HD; d += 128)
                *reinterpret_cast<uint32_t*>(kd + d) = pack2_bf16(rotated<HD>(kh, s_cs, d), rotated<HD>(kh, s_cs, d + 1));
            bf16_t* vd = f.v_out + (static_cast<int64_t>(page) * n_kv + kvh) * head_stride + off;
            for (int d = lane; d < HD; d += 64) vd[static_cast<int64_t>(d) * page_size] = from_float<bf16_t>(vh[d]);
        }
    };

    // QKV: the block table (warm in the L2) is read first, then the reads of the sums (which come from
    // further away) and of the first keys go out together; the queries are built from LDS while the keys
    // are under way
    if constexpr (ALL_AHEAD) {
        Where at[4];
        Block blk[4];
        auto locate4 = [&](int kb0) {
#pragma unroll
            for (int d = 0; d < 4; ++d) locate(kb0 + 32 * d, at[d]);  // past the end: page 0, masked below
        };
        auto load4 = [&]() {
#pragma unroll
            for (int d = 0; d < 4; ++d) load_block(at[d], blk[d]);
        };
        const bool any = !helper && kb_begin < kb_end;
        if (any) locate4(kb_begin);
        if (any) load4();
        if constexpr (QKV) {
            if (sums_here) {
                issue_sums();
                finish_sums();
            }
            __syncthreads();
            if (helper) return;
            build_queries();
            score_new_key();
        }
        for (int kb0 = kb_begin; kb0 < kb_end; kb0 += 4 * 32) {
            if (kb0 > kb_begin) {
                locate4(kb0);
                load4();
            }
#pragma unroll
            for (int d = 0; d < 4; ++d)
                if (kb0 + 32 * d < kb_end) compute_block(kb0 + 32 * d, blk[d]);
        }
    } else {
        const bool any = !helper && kb_begin < kb_end;
        Where at;
        Block cur, nxt;
        // (QKV: the reads of the sums, which come from further away than the table, go out before the
        // wait for the table)
        Asked first;
        if (any) ask_pages(kb_begin, first);
        if constexpr (QKV)
            if (sums_here) issue_sums();
        if (any) place(first, at);
        if (PREFETCH && any) {
            load_block(at, cur);
            locate(kb_begin + 32, at);
        }
        if constexpr (QKV) {
            if (sums_here) finish_sums();
            __syncthreads();
            if (helper) return;
            build_queries();
            score_new_key();
        }
        constexpr bool IN_TURN = QKV && MAXW <= 8;  // (16 waves a workgroup have 128 registers each: not enough)
        if (PREFETCH && any && !IN_TURN) {
            for (int kb = kb_begin; kb < kb_end; kb += 32) {
                if (kb + 32 < kb_end) {
                    load_block(at, nxt);
                    locate(kb + 64, at);
                }
                compute_block(kb, cur);
                cur = nxt;
            }
        } else if (PREFETCH && any) {
            // two blocks in turn, each in registers of its own: while one is computed the other's
            // data is under way (with one name for "this block" the copy from the next one's
            // registers at the end of a pass waits for that data).  A per cent of a step with long
            // contexts; the variants that would spill registers this way keep the loop above
            for (int kb = kb_begin;;) {
                if (kb + 32 < kb_end) {
                    load_block(at, nxt);
                    locate(kb + 64, at);
                }
                compute_block(kb, cur);
                kb += 32;
                if (kb >= kb_end) break;
                if (kb + 32 < kb_end) {
                    load_block(at, cur);
                    locate(kb + 64, at);
                }
                compute_block(kb, nxt);
                kb += 32;
                if (kb >= kb_end) break;
            }
        } else if (any) {
            for (int kb = kb_begin; kb < kb_end; kb += 32) {
                load_block(at, cur);
                locate(kb + 32, at);
                compute_block(kb, cur);
            }
        }
    }

    // ---- the denominator and maximum of every query row; several waves combine inside the
    // workgroup: maxima and sums through LDS, then the waves after the first lay their
    // accumulators, rescaled to the common maximum, into LDS, and the first wave adds them to its
    // own in the fixed order of the waves and writes the result (two barriers, no atomics)
    float l_tot[NT], m_fin[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        float l_w = l_run[nt];
        l_w = sum_xor32(sum_xor16(l_w));
        l_tot[nt] = l_w;
        m_fin[nt] = m_run[nt];
    }
    if (MAXW > 1 && n_waves > 1) {
        __shared__ float s_m[NT][MAXW][16], s_l[NT][MAXW][16];
        if (G == 0) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                s_m[nt][wave][c] = m_run[nt];
                s_l[nt][wave][c] = l_tot[nt];
            }
        }
        __syncthreads();
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float m_all = -INFINITY;
            for (int w = 0; w < n_runs; ++w) m_all = fmaxf(m_all, s_m[nt][w][c]);
            float denom = 0.f;
            for (int w = 0; w < n_runs; ++w) {
                const float mw = s_m[nt][w][c];
                if (mw != -INFINITY) denom += s_l[nt][w][c] * __builtin_amdgcn_exp2f(mw - m_all);
            }
            const float mine = (m_run[nt] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run[nt] - m_all);
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt) {
                acc[nt][dt][0] *= mine;
                acc[nt][dt][1] *= mine;
                acc[nt][dt][2] *= mine;
                acc[nt][dt][3] *= mine;
            }
            if (wave > 0 && wave < n_runs) {
#pragma unroll
                for (int dt = 0; dt < HDT; ++dt) s_o[(((wave - 1) * NT + nt) * HDT + dt) * 64 + lane] = acc[nt][dt];
            }
            l_tot[nt] = denom;
            m_fin[nt] = m_all;
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < n_runs; ++w) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int dt = 0; dt < HDT; ++dt) {
                    const floatx4 v = s_o[(((w - 1) * NT + nt) * HDT + dt) * 64 + lane];
                    acc[nt][dt][0] += v[0];
                    acc[nt][dt][1] += v[1];
                    acc[nt][dt][2] += v[2];
                    acc[nt][dt][3] += v[3];
                }
        }
    }

    // ---- results: lane holds O^T[d = 16 dt + 4 G + r][row c], relative to the maximum m_fin
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (!rvalid[nt]) continue;
        if (partial_base < 0) {
            const float inv = l_tot[nt] > 0.f ? 1.0f / l_tot[nt] : 0.f;
            bf16_t* o = out + (static_cast<int64_t>(q_row0 + rtok[nt]) * n_heads + rhead[nt]) * HD + 4 * G;
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt) {
                uint2 w;
                w.x = pack2_bf16(acc[nt][dt][0] * inv, acc[nt][dt][1] * inv);
                w.y = pack2_bf16(acc[nt][dt][2] * inv, acc[nt][dt][3] * inv);
                *reinterpret_cast<uint2*>(o + dt * 16) = w;
            }
        } else {
            // the item is one of several that share a query's keys: unnormalised sums, their
            // maximum (in natural units) and denominator, for attention_merge
            float* rec = partials + (static_cast<int64_t>(partial_base + rtok[nt]) * n_heads + rhead[nt]) * (HD + 2);
#pragma unroll
            for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) rec[dt * 16 + 4 * G + r] = acc[nt][dt][r];
            if (G == 0) {
                rec[HD] = m_fin[nt] * kLn2;
                rec[HD + 1] = l_tot[nt];
            }
        }
    }
}

template <int HDT, int NT>
int launch(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool, const int32_t* block_tables,
           int max_pages, const int32_t* items, int n_items, void* out, float* partials, int n_heads, int n_kv,
           int page_size, int window, float scale, int waves, hipStream_t stream) {
    constexpr int MAXW = NT == 1 ? max_waves<HDT>() : 4;
    const int group = n_heads / n_kv;
    const int rows = 16 * NT;
    const int gh = group < rows ? group : rows;
    const int head_chunks = (group + gh - 1) / gh;
    const dim3 grid(n_items, n_kv * head_chunks);
    if (waves < 1) waves = 1;
    if (waves > MAXW) waves = MAXW;
    // a launch of one wave per workgroup takes the instantiation without the LDS of the
    // combination, which would otherwise limit how many workgroups a compute unit holds
#define FSIE_ATTN_LAUNCH(W, THREADS, V)                                                                              \
    attention_mfma_kernel<HDT, NT, W, V><<<grid, THREADS, 0, stream>>>(                                              \
        static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool), \
        block_tables, max_pages, items, static_cast<bf16_t*>(out), partials, n_heads, n_kv, page_size, window, scale, \
        gh, head_chunks, QkvSums{})
    const bool v16 = page_size % 8 == 0;
    if (waves == 1) {
        if (v16) FSIE_ATTN_LAUNCH(1, 64, true);
        else FSIE_ATTN_LAUNCH(1, 64, false);
    } else {
        if (v16) FSIE_ATTN_LAUNCH(MAXW, 64 * waves, true);
        else FSIE_ATTN_LAUNCH(MAXW, 64 * waves, false);
    }
#undef FSIE_ATTN_LAUNCH
    FSIE_CHECK_LAUNCH("attention_mfma");
    return 0;
}

// The QKV variant: items of one token, head_dim a multiple of 32, page_size a multiple of 8.
template <int HDT>
int launch_qkv(const QkvSums& f, const void* k_pool, const void* v_pool, const int32_t* block_tables, int max_pages,
               const int32_t* items, int n_items, void* out, float* partials, int n_heads, int n_kv, int page_size,
               int window, float scale, int waves, hipStream_t stream) {
    constexpr int MAXW = max_waves<HDT>();
    const int group = n_heads / n_kv;
    const int gh = group < 16 ? group : 16;
    const int head_chunks = (group + gh - 1) / gh;
    const dim3 grid(n_items, n_kv * head_chunks);
    if (waves < 1) waves = 1;
    if (waves > MAXW) waves = MAXW;
#define FSIE_ATTN_LAUNCH(W, THREADS)                                                                                 \
    attention_mfma_kernel<HDT, 1, W, true, true><<<grid, THREADS, 0, stream>>>(                                      \
        nullptr, 0, static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool), block_tables, max_pages, \
        items, static_cast<bf16_t*>(out), partials, n_heads, n_kv, page_size, window, scale, gh, head_chunks, f)
    // one wave and three that only help with the sums; or all the waves the kernel has (those that an
    // item's keys leave idle help with the sums too)
    if (waves == 1) FSIE_ATTN_LAUNCH(1, 256);
    else FSIE_ATTN_LAUNCH(MAXW, 64 * MAXW);
#undef FSIE_ATTN_LAUNCH
    FSIE_CHECK_LAUNCH("attention_mfma_qkv");
    return 0;
}

typedef int (*LaunchQkvFn)(const QkvSums&, const void*, const void*, const int32_t*, int, const int32_t*, int, void*,
                           float*, int, int, int, int, float, int, hipStream_t);

typedef int (*LaunchFn)(const void*, int64_t, const void*, const void*, const int32_t*, int, const int32_t*, int, void*,
                        float*, int, int, int, int, float, int, hipStream_t);

}  // namespace fsie_attn
