// Attention over a paged cache whose keys and values differ in size (dim and vdim numbers per head), with soft-capped scores and a
// local mask: a query at position p reads the keys j <= p of its own chunk (j / chunk == p / chunk, chunks counted from position 0)
// and, with a window, j > p - window.  Scores, softmax and the weighted sum are float whatever the activation type.
//   k_plane [pages, kv_heads, page_size, dim], v_plane [pages, kv_heads, page_size, vdim]; key j of a request lies in slot
//   j % page_size of page block_table[request][j / page_size].
#include "common.h"

// ------------------------------------------------------------------ cache write
// Token t's keys and values go to their page; what would go to page 0 (the sentinel of rows that belong to no request) is dropped.
template <typename T>
__global__ void kv_cache_write_kernel(const T* __restrict__ k, int k_ld, const T* __restrict__ v, int v_ld, int kv_heads, int dim, int vdim,
                                      const int* __restrict__ token_req, const int* __restrict__ positions, const int* __restrict__ block_table,
                                      int table_ld, int table_width, T* __restrict__ k_plane, T* __restrict__ v_plane, int pages, int page_size) {
    const int t = blockIdx.x;
    const int p = positions[t], block = p / page_size;
    if (p < 0 || block >= table_width) return;
    const int page = block_table[(size_t)token_req[t] * table_ld + block];
    if (page <= 0 || page >= pages) return;
    const int slot = p % page_size;
    for (int i = threadIdx.x; i < kv_heads * dim; i += blockDim.x) {
        const int g = i / dim, d = i % dim;
        k_plane[(((size_t)page * kv_heads + g) * page_size + slot) * dim + d] = k[(size_t)t * k_ld + i];
    }
    for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x) {
        const int g = i / vdim, d = i % vdim;
        v_plane[(((size_t)page * kv_heads + g) * page_size + slot) * vdim + d] = v[(size_t)t * v_ld + i];
    }
}

extern "C" int tl_kv_cache_write(const void* k, int k_ld, const void* v, int v_ld, int tokens, int kv_heads, int dim, int vdim,
                                 const void* token_req, const void* positions, const void* block_table, int table_ld, int table_width,
                                 void* k_plane, void* v_plane, int pages, int page_size, int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && kv_heads > 0 && dim > 0 && vdim > 0 && page_size > 0 && pages > 0 && table_width > 0, "kv_cache_write: bad sizes");
    TL_REQUIRE(k_ld >= kv_heads * dim && v_ld >= kv_heads * vdim && table_ld >= table_width, "kv_cache_write: rows too short");
    if (tokens == 0) return TL_OK;
    if (dtype == TL_DT_F32)
        kv_cache_write_kernel<float><<<tokens, 256, 0, stream>>>((const float*)k, k_ld, (const float*)v, v_ld, kv_heads, dim, vdim, (const int*)token_req,
            (const int*)positions, (const int*)block_table, table_ld, table_width, (float*)k_plane, (float*)v_plane, pages, page_size);
    else if (dtype == TL_DT_BF16)
        kv_cache_write_kernel<bf16_t><<<tokens, 256, 0, stream>>>((const bf16_t*)k, k_ld, (const bf16_t*)v, v_ld, kv_heads, dim, vdim, (const int*)token_req,
            (const int*)positions, (const int*)block_table, table_ld, table_width, (bf16_t*)k_plane, (bf16_t*)v_plane, pages, page_size);
    else TL_REQUIRE(false, "kv_cache_write: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("kv_cache_write");
    return TL_OK;
}

// ------------------------------------------------------------------ the mask and the cap
struct LocalMask {
    int chunk, window;
    // the first key a query at position p reads
    __device__ __forceinline__ int first(int p) const {
        int lo = 0;
        if (chunk > 0) lo = max(lo, p / chunk * chunk);
        if (window > 0) lo = max(lo, p - window + 1);
        return lo;
    }
};

__device__ __forceinline__ float cap_score(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// ------------------------------------------------------------------ the general kernel
// One work-group of four waves per token and query head.  The keys lo .. p come in blocks of 64, dealt to the waves in turn (block b
// to wave b % 4: a matter of the position alone, so a token's result does not depend on the step it is in).  Within a block a lane
// owns a key: its score is the dot product with the query (kept in shared memory, scaled); the wave's running maximum and sum move on,
// and then a lane owns columns of the values: it adds p_j v_j over the block's keys, the weights read across the wave.  The four
// waves' states are joined in their order at the end.
#define LA_WAVES 4
#define LA_MAX_DIM 256
#define LA_COLS (LA_MAX_DIM / TL_WAVE)

template <typename T>
__global__ void __launch_bounds__(LA_WAVES * TL_WAVE)
local_attention_kernel(const T* __restrict__ q, int q_ld, T* __restrict__ out, int out_ld, const T* __restrict__ k_plane,
                       const T* __restrict__ v_plane, const int* __restrict__ block_table, int table_ld, const int* __restrict__ token_req,
                       const int* __restrict__ positions, int heads, int kv_heads, int dim, int vdim, int page_size, float scale, float cap,
                       LocalMask mask, float gain) {
    __shared__ float sq[LA_MAX_DIM];
    __shared__ float sm[LA_WAVES], sl[LA_WAVES];
    __shared__ float sacc[LA_WAVES][LA_MAX_DIM];
    const int t = blockIdx.x, head = blockIdx.y;
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    const int g = head / (heads / kv_heads);
    const int p = positions[t];
    const int lo = mask.first(p);
    const int* table = block_table + (size_t)token_req[t] * table_ld;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) sq[d] = to_float(q[(size_t)t * q_ld + head * dim + d]) * scale;
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[LA_COLS];
#pragma unroll
    for (int c = 0; c < LA_COLS; ++c) acc[c] = 0.f;
    const int nkeys = p - lo + 1;
    for (int b = wave; b * TL_WAVE < nkeys; b += LA_WAVES) {
        const int j = lo + b * TL_WAVE + lane;
        const bool ok = j <= p;
        float s = -INFINITY;
        size_t at = 0;                                 // the key's row in its plane, in rows of one head
        if (ok) {
            const int page = table[j / page_size];
            at = ((size_t)page * kv_heads + g) * page_size + j % page_size;
            const T* kr = k_plane + at * dim;
            float dot = 0.f;
            for (int d = 0; d < dim; ++d) dot = fmaf(sq[d], to_float(kr[d]), dot);
            s = cap_score(dot, cap);
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float w = ok ? expf(s - m_new) : 0.f;
        const float keep = expf(m - m_new);            // (0 for the first block: m = -inf)
        l = l * keep + wave_sum(w);
        m = m_new;
#pragma unroll
        for (int c = 0; c < LA_COLS; ++c) acc[c] *= keep;
        const int nb = min(TL_WAVE, p - (lo + b * TL_WAVE) + 1);
        for (int i = 0; i < nb; ++i) {
            const float wi = __shfl(w, i, TL_WAVE);
            const size_t ati = __shfl((unsigned long long)at, i, TL_WAVE);
            const T* vr = v_plane + ati * vdim;
#pragma unroll
            for (int c = 0; c < LA_COLS; ++c) {
                const int col = lane + c * TL_WAVE;
                if (col < vdim) acc[c] = fmaf(wi, to_float(vr[col]), acc[c]);
            }
        }
    }
    if (lane == 0) { sm[wave] = m; sl[wave] = l; }
#pragma unroll
    for (int c = 0; c < LA_COLS; ++c) sacc[wave][lane + c * TL_WAVE] = acc[c];
    __syncthreads();
    if (wave == 0) {
        float top = sm[0];
        for (int w = 1; w < LA_WAVES; ++w) top = fmaxf(top, sm[w]);
        float den = 0.f, f[LA_WAVES];
        for (int w = 0; w < LA_WAVES; ++w) {
            f[w] = sl[w] > 0.f ? expf(sm[w] - top) : 0.f;       // a wave without keys: no share
            den = fmaf(sl[w], f[w], den);
        }
        const float norm = gain / den;
        for (int col = lane; col < vdim; col += TL_WAVE) {
            float o = 0.f;
            for (int w = 0; w < LA_WAVES; ++w) o = fmaf(sacc[w][col], f[w], o);
            out[(size_t)t * out_ld + head * vdim + col] = from_float<T>(o * norm);
        }
    }
}

extern "C" int tl_local_attention(const void* q, int q_ld, void* out, int out_ld, const void* k_plane, const void* v_plane, int pages,
                                  const void* block_table, int table_ld, int table_width, const void* token_req, const void* positions,
                                  int tokens, int heads, int kv_heads, int dim, int vdim, int page_size, float scale, float cap, int chunk,
                                  int window, float gain, int longest, int general, int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && page_size > 0, "local_attention: bad sizes");
    TL_REQUIRE(dim <= LA_MAX_DIM && vdim <= LA_MAX_DIM, "local_attention: built for heads of up to %d numbers, got %d / %d", LA_MAX_DIM, dim, vdim);
    TL_REQUIRE(q_ld >= heads * dim && out_ld >= heads * vdim && table_ld >= table_width && chunk >= 0 && window >= 0, "local_attention: rows too short");
    TL_REQUIRE(heads <= 65535, "local_attention: too many heads");
    if (tokens == 0) return TL_OK;
    const LocalMask mask{chunk, window};
    dim3 grid(tokens, heads), block(LA_WAVES * TL_WAVE);
    if (dtype == TL_DT_F32)
        local_attention_kernel<float><<<grid, block, 0, stream>>>((const float*)q, q_ld, (float*)out, out_ld, (const float*)k_plane, (const float*)v_plane,
            (const int*)block_table, table_ld, (const int*)token_req, (const int*)positions, heads, kv_heads, dim, vdim, page_size, scale, cap, mask, gain);
    else if (dtype == TL_DT_BF16)
        local_attention_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)q, q_ld, (bf16_t*)out, out_ld, (const bf16_t*)k_plane, (const bf16_t*)v_plane,
            (const int*)block_table, table_ld, (const int*)token_req, (const int*)positions, heads, kv_heads, dim, vdim, page_size, scale, cap, mask, gain);
    else TL_REQUIRE(false, "local_attention: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("local_attention");
    return TL_OK;
}
