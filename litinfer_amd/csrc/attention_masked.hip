// Attention over the paged cache for mixers that the plain kernels do not cover: a window with a number of
// first positions that stay visible, scores capped by a tanh, keys and values of unequal sizes, and keys and
// values that are two column ranges of ONE cached row (a compressed cache: every query head reads the same
// row, the values are its first columns).  Queries are float32; scores, softmax and sums are float32.
// Beside it the per-head products that a compressed cache needs on both sides of the attention.
#include "common.h"

#define MA_MAX_CHUNKS 16          // value columns a lane sums: 64 * 16 = 1024

// The i-th visible key of the query at position p: first the kept ones (positions below min(keep, lo)),
// then lo .. p, with lo the window's lower edge.
__device__ __forceinline__ int visible_key(int i, int n_first, int lo) { return i < n_first ? i : lo + (i - n_first); }

// One wave per (token, query head).  A lane takes one key of a round of 64 for the scores (its row read in
// 16-byte pieces where the rows allow it), then one value column (and every 64th after it) for the sums.
template <typename T, typename TO, int NC, bool VEC>
__global__ __launch_bounds__(64) void masked_attention_wave_kernel(
    const float* __restrict__ q, int q_token_stride, int q_head_stride, TO* __restrict__ out,
    const T* __restrict__ kc, const T* __restrict__ vc, int k_row, int v_row,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ seg_of_token,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    int nh, int nkv, int dk, int dv, int page_size, int num_pages, int window, int keep_first, float softcap, float scale) {
    extern __shared__ float smem[];
    float* qs = smem;                        // [dk]
    float* ps = smem + dk;                   // [64]
    int* rowoff = (int*)(ps + LI_WAVE);      // [64]
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int s = seg_of_token[t];
    const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_first = keep_first < lo ? keep_first : lo;
    const int n_keys = n_first + (p - lo + 1);
    const int kvh = h / (nh / nkv);
    const int* table = block_table + (size_t)s * max_blocks;
    const float* qrow = q + (size_t)t * q_token_stride + (size_t)h * q_head_stride;
    for (int d = lane; d < dk; d += LI_WAVE) qs[d] = qrow[d];
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.f;
    for (int i0 = 0; i0 < n_keys; i0 += LI_WAVE) {
        const int i = i0 + lane;
        float sc = -INFINITY;
        int ro = -1;
        if (i < n_keys) {
            const int key = visible_key(i, n_first, lo);
            const int page = table[key / page_size];
            if (page >= 0 && page < num_pages) {
                ro = (page * nkv + kvh) * page_size + key % page_size;
                const T* krow = kc + (size_t)ro * k_row;
                float dot = 0.f;
                if constexpr (VEC) {
                    constexpr int E = 16 / sizeof(T);
                    for (int d = 0; d < dk; d += E) {
                        const uint4 raw = *reinterpret_cast<const uint4*>(krow + d);
                        if constexpr (sizeof(T) == 2) {
                            const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                dot = fmaf(qs[d + 2 * e], __uint_as_float(wv[e] << 16), dot);
                                dot = fmaf(qs[d + 2 * e + 1], __uint_as_float(wv[e] & 0xffff0000u), dot);
                            }
                        } else {
                            dot = fmaf(qs[d], __uint_as_float(raw.x), dot);
                            dot = fmaf(qs[d + 1], __uint_as_float(raw.y), dot);
                            dot = fmaf(qs[d + 2], __uint_as_float(raw.z), dot);
                            dot = fmaf(qs[d + 3], __uint_as_float(raw.w), dot);
                        }
                    }
                } else {
                    for (int d = 0; d < dk; ++d) dot = fmaf(qs[d], load_as_float(krow + d), dot);
                }
                sc = dot * scale;
                if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
            }
        }
        const float m_new = fmaxf(m, wave_max(sc));
        const float alpha = (l == 0.f) ? 0.f : expf(m - m_new);
        const float e = (ro >= 0) ? expf(sc - m_new) : 0.f;
        l = l * alpha + wave_sum(e);
        __syncthreads();
        ps[lane] = e;
        rowoff[lane] = ro;
        __syncthreads();
        const int nk = (n_keys - i0 < LI_WAVE) ? n_keys - i0 : LI_WAVE;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int d = lane + c * LI_WAVE;
            if (d < dv) {
                float a = acc[c] * alpha;
                for (int j = 0; j < nk; ++j) {
                    const int r = rowoff[j];
                    if (r >= 0) a = fmaf(ps[j], load_as_float(vc + (size_t)r * v_row + d), a);
                }
                acc[c] = a;
            }
        }
        m = m_new;
    }
    TO* orow = out + ((size_t)t * nh + h) * dv;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int d = lane + c * LI_WAVE;
        if (d < dv) store_from_float(orow + d, l != 0.f ? acc[c] / l : 0.f);
    }
}

template <typename T, typename TO, int NC>
static int launch_masked(const float* q, int qts, int qhs, void* out, const void* kc, const void* vc, int k_row, int v_row,
                         const int* block_table, int max_blocks, const int* seg_of_token, const int* q_start, const int* q_len,
                         const int* ctx_len, int T_, int nh, int nkv, int dk, int dv, int page_size, int num_pages, int window,
                         int keep_first, float softcap, float scale, hipStream_t stream) {
    const dim3 grid(T_, nh);
    const size_t lds = (size_t)(dk + 2 * LI_WAVE) * 4;
    constexpr int E = 16 / sizeof(T);
    const bool vec = dk % E == 0 && k_row % E == 0 && ((uintptr_t)kc % 16) == 0;
#define MA_GO(V)                                                                                                             \
    masked_attention_wave_kernel<T, TO, NC, V><<<grid, 64, lds, stream>>>(                                                   \
        q, qts, qhs, (TO*)out, (const T*)kc, (const T*)vc, k_row, v_row, block_table, max_blocks, seg_of_token, q_start,     \
        q_len, ctx_len, nh, nkv, dk, dv, page_size, num_pages, window, keep_first, softcap, scale)
    if (vec) MA_GO(true); else MA_GO(false);
#undef MA_GO
    return li_launch_status();
}

// q float32: head h of token t at q + t * q_token_stride + h * q_head_stride (dk values).  out [T, nh, dv] of
// out_dtype.  kc / vc: rows of k_row / v_row elements of cache_dtype, row (page * nkv + kv head) * page_size + place;
// the key is the first dk and the value the first dv elements of its row (the two may be the same memory).
extern "C" int li_masked_attention(const float* q, int q_token_stride, int q_head_stride, void* out, int out_dtype,
                                   const void* kc, const void* vc, int cache_dtype, int k_row, int v_row,
                                   const int* block_table, int max_blocks, const int* seg_of_token, const int* q_start,
                                   const int* q_len, const int* ctx_len, int T_, int nh, int nkv, int dk, int dv,
                                   int page_size, int num_pages, int window, int keep_first, float softcap, float scale,
                                   hipStream_t stream) {
    if (T_ <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dv <= 0 || dk > k_row || dv > v_row || page_size <= 0 ||
        window < 0 || keep_first < 0 || max_blocks <= 0 || nh > 65535 || dk > 8192 || dv > 64 * MA_MAX_CHUNKS)
        return LI_ERR_SIZE;
    const int nc = (dv + 63) / 64;
#define MA_ARGS q, q_token_stride, q_head_stride, out, kc, vc, k_row, v_row, block_table, max_blocks, seg_of_token, q_start, \
                q_len, ctx_len, T_, nh, nkv, dk, dv, page_size, num_pages, window, keep_first, softcap, scale, stream
#define MA_PICK(T, TO)                                                                  \
    {                                                                                   \
        if (nc <= 1) return launch_masked<T, TO, 1>(MA_ARGS);                           \
        if (nc <= 2) return launch_masked<T, TO, 2>(MA_ARGS);                           \
        if (nc <= 4) return launch_masked<T, TO, 4>(MA_ARGS);                           \
        if (nc <= 8) return launch_masked<T, TO, 8>(MA_ARGS);                           \
        return launch_masked<T, TO, MA_MAX_CHUNKS>(MA_ARGS);                            \
    }
    if (cache_dtype == LI_F32 && out_dtype == LI_F32) MA_PICK(float, float)
    if (cache_dtype == LI_BF16 && out_dtype == LI_BF16) MA_PICK(bf16_t, bf16_t)
    if (cache_dtype == LI_BF16 && out_dtype == LI_F32) MA_PICK(bf16_t, float)
#undef MA_PICK
#undef MA_ARGS
    return LI_ERR_DTYPE;
}

// ------------------------------------------------------------------------------------------- per-head products
// out[t, h, j] = sum_k m[h, j, k] * x[t, h, k]: every head has a matrix of its own, [n_out, n_in], stored one after
// the other.  x and out are addressed by a token stride and a head stride, so that a head's columns may lie inside
// a wider row.  A block takes one head, HL_TOK tokens and 256 outputs: the tokens' inputs lie in LDS as float32, a
// thread owns an output and reads its matrix row once for all the tokens.  Sums are float32, in the order of k.
#define HL_TOK 8

template <typename TX, typename TM, typename TO, bool VEC>
__global__ __launch_bounds__(256) void headwise_linear_kernel(
    const TX* __restrict__ x, long x_token_stride, int x_head_stride, const TM* __restrict__ m, TO* __restrict__ out,
    long o_token_stride, int o_head_stride, int T_, int n_out, int n_in) {
    extern __shared__ float xs[];                    // [HL_TOK][n_in]
    const int h = blockIdx.y, t0 = blockIdx.x * HL_TOK;
    const int nt = (T_ - t0 < HL_TOK) ? T_ - t0 : HL_TOK;
    for (int i = threadIdx.x; i < HL_TOK * n_in; i += 256) {
        const int tt = i / n_in, k = i % n_in;
        xs[i] = tt < nt ? load_as_float(x + (size_t)(t0 + tt) * x_token_stride + (size_t)h * x_head_stride + k) : 0.f;
    }
    __syncthreads();
    for (int j = blockIdx.z * 256 + threadIdx.x; j < n_out; j += gridDim.z * 256) {
        const TM* row = m + ((size_t)h * n_out + j) * n_in;
        float acc[HL_TOK];
#pragma unroll
        for (int tt = 0; tt < HL_TOK; ++tt) acc[tt] = 0.f;
        if constexpr (VEC) {
            constexpr int E = 16 / sizeof(TM);
            for (int k = 0; k < n_in; k += E) {
                const uint4 raw = *reinterpret_cast<const uint4*>(row + k);
                float wv[E];
                if constexpr (sizeof(TM) == 2) {
                    const uint32_t r4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        wv[2 * e] = __uint_as_float(r4[e] << 16);
                        wv[2 * e + 1] = __uint_as_float(r4[e] & 0xffff0000u);
                    }
                } else {
                    wv[0] = __uint_as_float(raw.x); wv[1] = __uint_as_float(raw.y);
                    wv[2] = __uint_as_float(raw.z); wv[3] = __uint_as_float(raw.w);
                }
#pragma unroll
                for (int e = 0; e < E; ++e)
#pragma unroll
                    for (int tt = 0; tt < HL_TOK; ++tt) acc[tt] = fmaf(wv[e], xs[tt * n_in + k + e], acc[tt]);
            }
        } else {
            for (int k = 0; k < n_in; ++k) {
                const float wv = load_as_float(row + k);
#pragma unroll
                for (int tt = 0; tt < HL_TOK; ++tt) acc[tt] = fmaf(wv, xs[tt * n_in + k], acc[tt]);
            }
        }
        for (int tt = 0; tt < nt; ++tt)
            store_from_float(out + (size_t)(t0 + tt) * o_token_stride + (size_t)h * o_head_stride + j, acc[tt]);
    }
}

extern "C" int li_headwise_linear(const void* x, int x_dtype, long x_token_stride, int x_head_stride, const void* m, int m_dtype,
                                  void* out, int out_dtype, long o_token_stride, int o_head_stride, int T_, int nh, int n_out,
                                  int n_in, hipStream_t stream) {
    if (T_ <= 0 || nh <= 0 || nh > 65535 || n_out <= 0 || n_in <= 0 || n_in > 2048) return LI_ERR_SIZE;
    const int zs = (n_out + 255) / 256;
    const dim3 grid((T_ + HL_TOK - 1) / HL_TOK, nh, zs < 64 ? zs : 64);
    const size_t lds = (size_t)HL_TOK * n_in * 4;
#define HL_GO(TX, TM, TO)                                                                                                  \
    {                                                                                                                      \
        constexpr int E = 16 / sizeof(TM);                                                                                 \
        if (n_in % E == 0 && ((uintptr_t)m % 16) == 0)                                                                     \
            headwise_linear_kernel<TX, TM, TO, true><<<grid, 256, lds, stream>>>(                                          \
                (const TX*)x, x_token_stride, x_head_stride, (const TM*)m, (TO*)out, o_token_stride, o_head_stride, T_, n_out, n_in); \
        else                                                                                                               \
            headwise_linear_kernel<TX, TM, TO, false><<<grid, 256, lds, stream>>>(                                         \
                (const TX*)x, x_token_stride, x_head_stride, (const TM*)m, (TO*)out, o_token_stride, o_head_stride, T_, n_out, n_in); \
        return li_launch_status();                                                                                         \
    }
    if (x_dtype == LI_F32 && m_dtype == LI_F32 && out_dtype == LI_F32) HL_GO(float, float, float)
    if (x_dtype == LI_F32 && m_dtype == LI_BF16 && out_dtype == LI_F32) HL_GO(float, bf16_t, float)
    if (x_dtype == LI_F32 && m_dtype == LI_BF16 && out_dtype == LI_BF16) HL_GO(float, bf16_t, bf16_t)
    if (x_dtype == LI_BF16 && m_dtype == LI_BF16 && out_dtype == LI_BF16) HL_GO(bf16_t, bf16_t, bf16_t)
    if (x_dtype == LI_BF16 && m_dtype == LI_BF16 && out_dtype == LI_F32) HL_GO(bf16_t, bf16_t, float)
#undef HL_GO
    return LI_ERR_DTYPE;
}
