// Causal grouped-query attention over the pages of the cache: float32 arithmetic throughout
// (products, softmax, sums), for float32 or bfloat16 storage.  It is the attention of the 32-bit
// path and takes any head size up to 256.
//
// The host cuts the step into work items (api.h: FSIE_ATTN_ITEM_*): a tile of up to 16/gh query
// tokens of one request, a range of keys, and where the result goes: the output (normalised), or a
// partial record (unnormalised sum, running maximum, denominator) that attention_merge combines
// when a key range was split over several items.  grid = (items, kv_heads * head_chunks); a block
// holds rows = tokens x heads of one kv head's group (gh heads per chunk), four rows per wave.
//
// Page layout: keys [page][kv_head][slot][head_dim], values [page][kv_head][head_dim][slot]; block_tables[seq * max_pages + i] = page id of the
// request's i-th page, or -1 where a window has passed.
#include "common.h"
#include "api.h"

#include <math.h>

namespace {

constexpr int kRows = 16;      // query rows per block
constexpr int kKeys = 32;      // keys per tile
constexpr int kMaxChunks = 8;  // head_dim <= 32 * 8

__device__ __forceinline__ float half_wave_max(float v) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, FSIE_WAVE));
    return v;
}
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, FSIE_WAVE);
    return v;
}

// Four consecutive elements as floats: one 16-byte (float32) or 8-byte (bfloat16) load.
__device__ __forceinline__ void load4(const float* p, float (&f)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&f)[4]) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    f[0] = __uint_as_float(v.x << 16), f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16), f[3] = __uint_as_float(v.y & 0xffff0000u);
}

// VEC: the head size and the page size are multiples of 4 and the pools are aligned for load4, so a
// thread copies four values of a key (along the head) or of a dimension (four consecutive slots of a
// page; only for items whose first key is a multiple of 4, else element by element) with one load.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void attention_scalar_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_pages, const int32_t* __restrict__ items,
    T* __restrict__ out, float* __restrict__ partials, int n_heads, int n_kv, int hd, int page_size,
    int window, float scale, int gh, int head_chunks) {
    extern __shared__ float lds[];
    float* qs = lds;                          // [kRows][hd]
    float* kv = qs + kRows * hd;              // [kKeys][hd + 1]
    float* ps = kv + kKeys * (hd + 1);        // [kRows][kKeys]
    const int kv_stride = hd + 1;

    const int32_t* item = items + static_cast<int64_t>(blockIdx.x) * FSIE_ATTN_ITEM_INTS;
    const int seq = item[FSIE_ATTN_ITEM_SEQ];
    const int q_row0 = item[FSIE_ATTN_ITEM_QROW];
    const int n_q = item[FSIE_ATTN_ITEM_NQ];
    const int pos0 = item[FSIE_ATTN_ITEM_POS];
    const int key_begin = item[FSIE_ATTN_ITEM_KBEGIN];
    const int key_end = item[FSIE_ATTN_ITEM_KEND];
    const int partial_base = item[FSIE_ATTN_ITEM_PARTIAL];
    if (n_q <= 0) return;  // padding item

    const int group = n_heads / n_kv;
    const int kvh = blockIdx.y / head_chunks;
    const int chunk = blockIdx.y - kvh * head_chunks;
    const int gh_here = min(gh, group - chunk * gh);
    const int h_base = kvh * group + chunk * gh;
    const int n_rows = n_q * gh;

    const int tid = threadIdx.x;
    const int lane = tid & (FSIE_WAVE - 1);
    const int wave = tid / FSIE_WAVE;
    const int sub = lane >> 5;    // which of the two rows of a pass
    const int lane32 = lane & 31;

    // queries of this block's rows
    for (int e = tid; e < kRows * hd; e += blockDim.x) {
        const int r = e / hd, d = e - r * hd;
        float v = 0.f;
        if (r < n_rows && (r % gh) < gh_here) {
            const int tq = r / gh, hq = h_base + (r % gh);
            v = to_float(q[static_cast<int64_t>(q_row0 + tq) * q_stride + static_cast<int64_t>(hq) * hd + d]);
        }
        qs[e] = v;
    }

    float m_run[2], l_run[2], acc[2][kMaxChunks];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        m_run[p] = -INFINITY;
        l_run[p] = 0.f;
#pragma unroll
        for (int i = 0; i < kMaxChunks; ++i) acc[p][i] = 0.f;
    }
    const int n_chunks = (hd + 31) / 32;
    const int32_t* table = block_tables + static_cast<int64_t>(seq) * max_pages;

    const bool slots_by_four = VEC && (key_begin & 3) == 0;
    for (int kt = key_begin; kt < key_end; kt += kKeys) {
        __syncthreads();  // previous tile's values are no longer read (first pass: qs is written)
        if (VEC) {
            const int per_key = hd >> 2;
            for (int e = tid; e < kKeys * per_key; e += blockDim.x) {
                const int j = e / per_key, d = (e - j * per_key) * 4;
                const int kj = kt + j;
                float f[4] = {0.f, 0.f, 0.f, 0.f};
                if (kj < key_end) {
                    const int page = table[kj / page_size];
                    if (page >= 0)
                        load4(k_pool + ((static_cast<int64_t>(page) * n_kv + kvh) * page_size + kj % page_size) * hd + d, f);
                }
                float* dst = kv + j * kv_stride + d;
                dst[0] = f[0], dst[1] = f[1], dst[2] = f[2], dst[3] = f[3];
            }
        } else {
            for (int e = tid; e < kKeys * hd; e += blockDim.x) {
                const int j = e / hd, d = e - j * hd;
                const int kj = kt + j;
                float v = 0.f;
                if (kj < key_end) {
                    const int page = table[kj / page_size];
                    if (page >= 0) {
                        v = to_float(k_pool[((static_cast<int64_t>(page) * n_kv + kvh) * page_size + kj % page_size) * hd + d]);
                    }
                }
                kv[j * kv_stride + d] = v;
            }
        }
        __syncthreads();
        float corr[2];
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int r = wave * 4 + p * 2 + sub;
            const bool row_ok = r < n_rows && (r % gh) < gh_here;
            const int pos = pos0 + r / gh;
            const int kj = kt + lane32;
            bool visible = row_ok && kj < key_end && kj <= pos && (window <= 0 || kj > pos - window);
            if (visible) visible = table[kj / page_size] >= 0;
            float s = -INFINITY;
            if (visible) {
                const float* qr = qs + r * hd;
                const float* kr = kv + lane32 * kv_stride;
                float dot = 0.f;
                for (int d = 0; d < hd; ++d) dot = fmaf(qr[d], kr[d], dot);
                s = dot * scale;
            }
            const float m_new = fmaxf(m_run[p], half_wave_max(s));
            const float pe = (s == -INFINITY) ? 0.f : expf(s - m_new);
            corr[p] = (m_run[p] == -INFINITY) ? 1.f : expf(m_run[p] - m_new);
            l_run[p] = l_run[p] * corr[p] + half_wave_sum(pe);
            m_run[p] = m_new;
            ps[r * kKeys + lane32] = pe;
        }
        __syncthreads();  // scores done: the tile buffer can take the values
        if (slots_by_four) {
            // a page of values is [head_dim][page_size]: consecutive threads take the eight groups of
            // four keys of a dimension, then the next dimension
            for (int e = tid; e < (kKeys / 4) * hd; e += blockDim.x) {
                const int g = e & (kKeys / 4 - 1), d = e / (kKeys / 4);
                const int kj = kt + 4 * g;  // a multiple of 4: the four slots lie in one page
                float f[4] = {0.f, 0.f, 0.f, 0.f};
                if (kj < key_end) {
                    const int page = table[kj / page_size];
                    if (page >= 0)
                        load4(v_pool + ((static_cast<int64_t>(page) * n_kv + kvh) * hd + d) * page_size + kj % page_size, f);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) kv[(4 * g + t) * kv_stride + d] = kj + t < key_end ? f[t] : 0.f;
            }
        } else {
            for (int e = tid; e < kKeys * hd; e += blockDim.x) {
                const int j = e / hd, d = e - j * hd;
                const int kj = kt + j;
                float v = 0.f;
                if (kj < key_end) {
                    const int page = table[kj / page_size];
                    if (page >= 0) {
                        v = to_float(v_pool[((static_cast<int64_t>(page) * n_kv + kvh) * hd + d) * page_size + kj % page_size]);
                    }
                }
                kv[j * kv_stride + d] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int r = wave * 4 + p * 2 + sub;
            const float* pr = ps + r * kKeys;
#pragma unroll
            for (int i = 0; i < kMaxChunks; ++i) {
                if (i < n_chunks) {
                    const int d = lane32 + 32 * i;
                    float a = acc[p][i] * corr[p];
                    if (d < hd) {
                        for (int j = 0; j < kKeys; ++j) a = fmaf(pr[j], kv[j * kv_stride + d], a);
                    }
                    acc[p][i] = a;
                }
            }
        }
    }

    // results
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int r = wave * 4 + p * 2 + sub;
        if (!(r < n_rows && (r % gh) < gh_here)) continue;
        const int tq = r / gh, hq = h_base + (r % gh);
        if (partial_base < 0) {
            const float inv = l_run[p] > 0.f ? 1.0f / l_run[p] : 0.f;
            T* o = out + (static_cast<int64_t>(q_row0 + tq) * n_heads + hq) * hd;
#pragma unroll
            for (int i = 0; i < kMaxChunks; ++i) {
                const int d = lane32 + 32 * i;
                if (i < n_chunks && d < hd) o[d] = from_float<T>(acc[p][i] * inv);
            }
        } else {
            float* rec = partials + (static_cast<int64_t>(partial_base + tq) * n_heads + hq) * (hd + 2);
#pragma unroll
            for (int i = 0; i < kMaxChunks; ++i) {
                const int d = lane32 + 32 * i;
                if (i < n_chunks && d < hd) rec[d] = acc[p][i];
            }
            if (lane32 == 0) {
                rec[hd] = m_run[p];
                rec[hd + 1] = l_run[p];
            }
        }
    }
}

// Combine the partial records of one query token in the fixed order of its splits.
// merge item: {out_row, first_slot, n_splits, slot_stride}
// One workgroup per (token, head).  Up to kMergeWideFrom splits are one wave's work (the other
// three leave at once): the maxima and denominators of up to 64 splits are read by one lane each,
// and the sums of a dimension are loaded several splits ahead of their use: a loop that waits for
// each record in turn costs a memory latency per split (28 splits took longer than the attention
// itself).  More splits (one request of 100,000 keys is cut into more than a hundred items) are
// dealt to the four waves in runs, which add their sums up through LDS in the order of the waves.
constexpr int kMergeWideFrom = 32;

template <typename T, int DIMS>
__global__ __launch_bounds__(256) void attention_merge_kernel(const float* __restrict__ partials,
                                                              const int32_t* __restrict__ merges, T* __restrict__ out,
                                                              int n_heads, int hd) {
    __shared__ float handed[3][DIMS * 64 + 1];  // of waves 1 to 3: the sums, then the denominator
    const int32_t* mi = merges + static_cast<int64_t>(blockIdx.x) * FSIE_ATTN_MERGE_INTS;
    const int out_row = mi[0], first = mi[1], n_splits = mi[2], stride = mi[3];
    if (n_splits <= 0) return;
    const int hq = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const bool wide = n_splits > kMergeWideFrom;  // the same for the whole workgroup
    if (!wide && wave > 0) return;
    const int64_t rec_size = hd + 2;
    const float* rec0 = partials + (static_cast<int64_t>(first) * n_heads + hq) * rec_size;
    const int64_t rec_step = static_cast<int64_t>(stride) * n_heads * rec_size;
    constexpr int AHEAD = 8;
    float denom = 0.f;  // summed in the order of the splits, as the accumulators are
    float a[DIMS];
#pragma unroll
    for (int i = 0; i < DIMS; ++i) a[i] = 0.f;
    if (n_splits <= AHEAD) {
        // few splits (a decode step's usual case): maxima, denominators and sums are all asked for
        // at once, one trip to memory instead of two; the arithmetic and its order are those of
        // the general case below
        const int s = min(lane, n_splits - 1);
        const float ms = rec0[s * rec_step + hd];
        const float l = rec0[s * rec_step + hd + 1];
        float v[AHEAD][DIMS];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            const float* r = rec0 + min(j, n_splits - 1) * rec_step;
#pragma unroll
            for (int i = 0; i < DIMS; ++i) v[j][i] = r[min(lane + 64 * i, hd - 1)];
        }
        const float m = wave_max(lane < n_splits ? ms : -INFINITY);
        const float w = (lane >= n_splits || ms == -INFINITY) ? 0.f : expf(ms - m);
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            const float wj = j < n_splits ? __shfl(w, j) : 0.f;
            const float lj = __shfl(l, j);
            if (wj != 0.f) {  // the same for the whole wave
                denom += lj * wj;
#pragma unroll
                for (int i = 0; i < DIMS; ++i) a[i] += v[j][i] * wj;
            }
        }
    } else {
        float m = -INFINITY;  // over all splits, in every wave
        for (int base = 0; base < n_splits; base += 64) {
            const int s = base + lane;
            m = fmaxf(m, s < n_splits ? rec0[s * rec_step + hd] : -INFINITY);
        }
        m = wave_max(m);
        // this wave's run of the splits: all of them, or a quarter
        int s_begin = 0, s_end = n_splits;
        if (wide) {
            const int run = (n_splits + 3) / 4;
            s_begin = wave * run;
            s_end = min(n_splits, s_begin + run);
        }
        for (int base = s_begin; base < s_end; base += 64) {
            const int s = base + lane;
            float w = 0.f, l = 0.f;
            if (s < s_end) {
                const float ms = rec0[s * rec_step + hd];
                l = rec0[s * rec_step + hd + 1];
                w = ms == -INFINITY ? 0.f : expf(ms - m);
            }
            const int here = min(64, s_end - base);
            const float* rec = rec0 + base * rec_step;
            for (int j0 = 0; j0 < here; j0 += AHEAD) {
                float v[AHEAD][DIMS];
#pragma unroll
                for (int j = 0; j < AHEAD; ++j) {  // a split past the end reads the last one again, with weight 0
                    const float* r = rec + min(j0 + j, here - 1) * rec_step;
#pragma unroll
                    for (int i = 0; i < DIMS; ++i) v[j][i] = r[min(lane + 64 * i, hd - 1)];
                }
#pragma unroll
                for (int j = 0; j < AHEAD; ++j) {
                    const int src = min(j0 + j, 63);
                    const float wj = j0 + j < here ? __shfl(w, src) : 0.f;
                    const float lj = __shfl(l, src);
                    if (wj != 0.f) {  // the same for the whole wave
                        denom += lj * wj;
#pragma unroll
                        for (int i = 0; i < DIMS; ++i) a[i] += v[j][i] * wj;
                    }
                }
            }
        }
    }
    if (wide) {
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < DIMS; ++i) handed[wave - 1][i * 64 + lane] = a[i];
            if (lane == 0) handed[wave - 1][DIMS * 64] = denom;
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            denom += handed[w][DIMS * 64];
#pragma unroll
            for (int i = 0; i < DIMS; ++i) a[i] += handed[w][i * 64 + lane];
        }
    }
    const float inv = denom > 0.f ? 1.0f / denom : 0.f;
#pragma unroll
    for (int i = 0; i < DIMS; ++i) {
        const int d = lane + 64 * i;
        if (d < hd) out[(static_cast<int64_t>(out_row) * n_heads + hq) * hd + d] = from_float<T>(a[i] * inv);
    }
}

template <typename T>
void launch_merge(const float* partials, const int32_t* merges, int n_merges, T* out, int n_heads, int hd,
                  hipStream_t stream) {
    const dim3 grid(n_merges, n_heads);
    if (hd <= 64) attention_merge_kernel<T, 1><<<grid, 256, 0, stream>>>(partials, merges, out, n_heads, hd);
    else if (hd <= 128) attention_merge_kernel<T, 2><<<grid, 256, 0, stream>>>(partials, merges, out, n_heads, hd);
    else attention_merge_kernel<T, 4><<<grid, 256, 0, stream>>>(partials, merges, out, n_heads, hd);
}

}  // namespace

extern "C" int fsie_attention_scalar(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                                     const int32_t* block_tables, int max_pages, const int32_t* items,
                                     int n_items, void* out, float* partials, int n_heads, int n_kv,
                                     int head_dim, int page_size, int window, float scale, int dtype,
                                     hipStream_t stream) {
    FSIE_REQUIRE(n_items >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0,
                 "attention: heads %d must be a positive multiple of kv heads %d", n_heads, n_kv);
    FSIE_REQUIRE(head_dim > 0 && head_dim <= 32 * kMaxChunks, "attention: head_dim %d must be in 1..%d",
                 head_dim, 32 * kMaxChunks);
    FSIE_REQUIRE(page_size > 0 && max_pages > 0, "attention: bad page geometry");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "attention: unknown dtype %d", dtype);
    if (n_items == 0) return 0;
    const int group = n_heads / n_kv;
    const int gh = group < kRows ? group : kRows;
    const int head_chunks = (group + gh - 1) / gh;
    const dim3 grid(n_items, n_kv * head_chunks);
    const size_t lds = sizeof(float) * (static_cast<size_t>(kRows) * head_dim + kKeys * (head_dim + 1) + kRows * kKeys);
    const bool vec = head_dim % 4 == 0 && page_size % 4 == 0 && reinterpret_cast<uintptr_t>(k_pool) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(v_pool) % 16 == 0;
    if (dtype == FSIE_F32) {
        auto kernel = vec ? attention_scalar_kernel<float, true> : attention_scalar_kernel<float, false>;
        kernel<<<grid, 256, lds, stream>>>(
            static_cast<const float*>(q), q_stride, static_cast<const float*>(k_pool), static_cast<const float*>(v_pool),
            block_tables, max_pages, items, static_cast<float*>(out), partials, n_heads, n_kv, head_dim, page_size,
            window, scale, gh, head_chunks);
    } else {
        auto kernel = vec ? attention_scalar_kernel<bf16_t, true> : attention_scalar_kernel<bf16_t, false>;
        kernel<<<grid, 256, lds, stream>>>(
            static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(k_pool),
            static_cast<const bf16_t*>(v_pool), block_tables, max_pages, items, static_cast<bf16_t*>(out), partials,
            n_heads, n_kv, head_dim, page_size, window, scale, gh, head_chunks);
    }
    FSIE_CHECK_LAUNCH("attention_scalar");
    return 0;
}

extern "C" int fsie_attention_merge(const float* partials, const int32_t* merges, int n_merges, void* out,
                                    int n_heads, int head_dim, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_merges >= 0 && n_heads > 0 && head_dim > 0, "attention_merge: bad sizes");
    FSIE_REQUIRE(head_dim <= 256, "attention_merge: head_dim %d is larger than 256", head_dim);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "attention_merge: unknown dtype %d", dtype);
    if (n_merges == 0) return 0;
    if (dtype == FSIE_F32) launch_merge(partials, merges, n_merges, static_cast<float*>(out), n_heads, head_dim, stream);
    else launch_merge(partials, merges, n_merges, static_cast<bf16_t*>(out), n_heads, head_dim, stream);
    FSIE_CHECK_LAUNCH("attention_merge");
    return 0;
}

// Query tokens per work item for a model with `n_heads` and `n_kv` heads, so that the host cuts
// tiles the way the kernel expects.
extern "C" int fsie_attention_scalar_tile_tokens(int n_heads, int n_kv) {
    if (n_kv <= 0 || n_heads <= 0 || n_heads % n_kv) return 0;
    const int group = n_heads / n_kv;
    const int gh = group < kRows ? group : kRows;
    return kRows / gh;
}
