// Attention over a cached latent: every token keeps one row of `rank` normed latent numbers followed by `rot`
// rotated key numbers that all heads share.  A head's query is brought into the same shape beforehand (its
// unrotated part multiplied through the key up-projection, its rotated part turned by its position), so a
// score is one dot product of rank + rot numbers and the weighted sum runs over the latent rows themselves;
// the value up-projection follows outside.  Norms, angles, scores, weights and sums are float.
#include "common.h"

// The pair (u, v) at entries (2i, 2i + 1) turned by position * inv_freq[i].
__device__ __forceinline__ void turn_pair(float u, float v, float pos, float f, float& a, float& b) {
    float s, c;
    sincosf(pos * f, &s, &c);
    a = u * c - v * s;
    b = v * c + u * s;
}

// ------------------------------------------------------------------ norms of the two latents, rotation, cache write
// down [tokens, ld]: q_rank numbers of the query latent, then rank of the key/value latent, then rot of the shared key part.
// cq = rmsnorm(first q_rank) * wq;  page row of the token = [rmsnorm(next rank) * wkv, the last rot with the first
// rot_dims of them turned in pairs].  A token whose block-table entry is 0 (the sentinel page) writes nothing.
template <typename T>
__global__ void latent_prepare_kernel(const T* __restrict__ down, int ld, int q_rank, int rank, int rot, int rot_dims,
                                      const void* __restrict__ wq, int wq_f32, const void* __restrict__ wkv, int wkv_f32, float eps,
                                      const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                      const int* __restrict__ token_req, const int* __restrict__ block_table, int bt_stride,
                                      T* __restrict__ plane, int page_size, T* __restrict__ cq) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const T* row = down + (size_t)t * ld;
    float ss = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) { const float x = to_float(row[i]); ss = fmaf(x, x, ss); }
    ss = block_sum(ss, red);
    float inv = 1.f / sqrtf(ss / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
        cq[(size_t)t * q_rank + i] = from_float<T>(to_float(row[i]) * inv * load_vec(wq, wq_f32, i));
    if (plane == nullptr) return;
    const int pos = positions[t];
    const int page = block_table[(size_t)token_req[t] * bt_stride + pos / page_size];
    ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) { const float x = to_float(row[q_rank + i]); ss = fmaf(x, x, ss); }
    ss = block_sum(ss, red);
    if (page == 0) return;
    inv = 1.f / sqrtf(ss / (float)rank + eps);
    T* dst = plane + ((size_t)page * page_size + pos % page_size) * (rank + rot);
    for (int i = threadIdx.x; i < rank; i += blockDim.x)
        dst[i] = from_float<T>(to_float(row[q_rank + i]) * inv * load_vec(wkv, wkv_f32, i));
    const T* kr = row + q_rank + rank;
    for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
        float a, b;
        turn_pair(to_float(kr[2 * i]), to_float(kr[2 * i + 1]), (float)pos, inv_freq[i], a, b);
        dst[rank + 2 * i] = from_float<T>(a);
        dst[rank + 2 * i + 1] = from_float<T>(b);
    }
    for (int i = rot_dims + threadIdx.x; i < rot; i += blockDim.x) dst[rank + i] = kr[i];
}

extern "C" int tl_latent_prepare(const void* down, int ld, int q_rank, int rank, int rot, int rot_dims, const void* wq, int wq_f32,
                                 const void* wkv, int wkv_f32, float eps, const void* positions, const void* inv_freq,
                                 const void* token_req, const void* block_table, int bt_stride, void* plane, int page_size,
                                 void* cq, int tokens, int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && q_rank > 0 && rank > 0 && rot >= 0 && rot_dims % 2 == 0 && rot_dims <= rot && ld >= q_rank + rank + rot,
               "latent_prepare: bad sizes");
    TL_REQUIRE(plane == nullptr || (page_size > 0 && block_table != nullptr && token_req != nullptr), "latent_prepare: a cache write needs the block table");
    if (tokens == 0) return TL_OK;
    dim3 grid(tokens), block(256);
#define TL_ARGS(T) (const T*)down, ld, q_rank, rank, rot, rot_dims, wq, wq_f32, wkv, wkv_f32, eps, (const int*)positions, (const float*)inv_freq, \
                   (const int*)token_req, (const int*)block_table, bt_stride, (T*)plane, page_size, (T*)cq
    if (dtype == TL_DT_F32) latent_prepare_kernel<float><<<grid, block, 0, stream>>>(TL_ARGS(float));
    else if (dtype == TL_DT_BF16) latent_prepare_kernel<bf16_t><<<grid, block, 0, stream>>>(TL_ARGS(bf16_t));
    else TL_REQUIRE(false, "latent_prepare: unknown dtype %d", dtype);
#undef TL_ARGS
    TL_CHECK_LAUNCH("latent_prepare");
    return TL_OK;
}

// ------------------------------------------------------------------ rotated query parts into place
// dst[t, h, dst_off + i] = the entries src[t, h, src_off + i], i < rot, the first rot_dims of them turned in pairs.
template <typename T>
__global__ void rotate_pairs_kernel(const T* src, int src_ld, int src_head, int src_off,       // (src may be dst: a thread reads its
                                    T* dst, int dst_ld, int dst_head, int dst_off,               // pair before it writes it)
                                    const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                    int heads, int rot, int rot_dims) {
    const int t = blockIdx.x;
    const float pos = (float)positions[t];
    const int half = rot_dims / 2, tail = rot - rot_dims;
    for (int i = threadIdx.x; i < heads * (half + tail); i += blockDim.x) {
        const int h = i / (half + tail), j = i % (half + tail);
        const T* s = src + (size_t)t * src_ld + h * src_head + src_off;
        T* d = dst + (size_t)t * dst_ld + h * dst_head + dst_off;
        if (j < half) {
            float a, b;
            turn_pair(to_float(s[2 * j]), to_float(s[2 * j + 1]), pos, inv_freq[j], a, b);
            d[2 * j] = from_float<T>(a);
            d[2 * j + 1] = from_float<T>(b);
        } else {
            d[rot_dims + j - half] = s[rot_dims + j - half];
        }
    }
}

extern "C" int tl_rotate_pairs(const void* src, int src_ld, int src_head, int src_off, void* dst, int dst_ld, int dst_head, int dst_off,
                               const void* positions, const void* inv_freq, int tokens, int heads, int rot, int rot_dims, int dtype,
                               hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && heads > 0 && rot >= 0 && rot_dims % 2 == 0 && rot_dims <= rot, "rotate_pairs: bad sizes");
    if (tokens == 0 || rot == 0) return TL_OK;
    dim3 grid(tokens), block(256);
    if (dtype == TL_DT_F32)
        rotate_pairs_kernel<float><<<grid, block, 0, stream>>>((const float*)src, src_ld, src_head, src_off, (float*)dst, dst_ld, dst_head, dst_off,
                                                               (const int*)positions, (const float*)inv_freq, heads, rot, rot_dims);
    else if (dtype == TL_DT_BF16)
        rotate_pairs_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)src, src_ld, src_head, src_off, (bf16_t*)dst, dst_ld, dst_head, dst_off,
                                                                (const int*)positions, (const float*)inv_freq, heads, rot, rot_dims);
    else TL_REQUIRE(false, "rotate_pairs: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("rotate_pairs");
    return TL_OK;
}

// ------------------------------------------------------------------ attention
// A tile is up to `tile_tokens` consecutive new tokens of one request times a chunk of up to 16 heads: one wave per
// row (token, head).  The keys pass through shared memory KT at a time, shared by all rows of the tile; a lane takes the
// score of one key (a dot product of rank + rot numbers), the wave takes maximum and sum, then the lanes take the
// latent's columns for the weighted sum.  The softmax runs online and starts from the sink: maximum = sink, sum = 1,
// which is the sink's own term exp(sink - sink) with no value behind it (without a sink: -inf and 0).
// With splits > 1 the keys of a tile are dealt to that many work-groups in turns of KT keys; each leaves its sums,
// maximum and denominator, and a second kernel merges them (the sink counts in part 0 only).
#define LAT_KT 32
#define LAT_ROWS 16

template <typename T>
__global__ void __launch_bounds__(LAT_ROWS * TL_WAVE)
latent_attention_kernel(const T* __restrict__ q, int q_ld, T* __restrict__ out, const T* __restrict__ plane,
                        const int* __restrict__ block_table, int bt_stride, const int* __restrict__ req_indptr,
                        const int* __restrict__ ctx_lens, const int* __restrict__ tile_req, const int* __restrict__ tile_tok0,
                        int tile_tokens, int heads, int rank, int rot, int page_size, float scale, const float* __restrict__ sink,
                        int splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
    extern __shared__ float smem[];
    const int D = rank + rot, ldk = D + 1;             // a row more than a multiple of the banks apart: lanes read rows side by side
    float* sk = smem;                                  // [KT][ldk]
    float* sq = sk + LAT_KT * ldk;                     // [rows][D]
    float* sp = sq + LAT_ROWS * D;                     // [rows][KT]
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    const int tile = blockIdx.x, head0 = blockIdx.y * LAT_ROWS, split = blockIdx.z;
    const int hchunk = min(LAT_ROWS, heads - head0);
    const int req = tile_req ? tile_req[tile] : tile, tok0 = tile_req ? tile_tok0[tile] : 0;
    const int first = req_indptr ? req_indptr[req] : req, n_new = req_indptr ? req_indptr[req + 1] - first : 1;
    const int ctx = ctx_lens[req];
    const int ntok = min(tile_tokens, n_new - tok0);
    const int rows = ntok * hchunk;
    // row of this wave
    const bool row_ok = wave < rows;
    const int rt = row_ok ? wave / hchunk : 0, rh = row_ok ? head0 + wave % hchunk : head0;
    const int tok = first + tok0 + rt;                 // index of the row's token in the step
    const int qpos = ctx + tok0 + rt;                  // its position: it sees the keys 0 .. qpos
    if (row_ok) {
        const T* qr = q + (size_t)tok * q_ld + (size_t)rh * D;
        for (int i = lane; i < D; i += TL_WAVE) sq[wave * D + i] = to_float(qr[i]);
    }
    const int cols = (rank + TL_WAVE - 1) / TL_WAVE;    // latent columns a lane sums (at most 16: rank <= 1024)
    float acc[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[c] = 0.f;
    const bool with_sink = sink != nullptr && split == 0;
    float m = with_sink ? sink[rh] : -INFINITY, l = with_sink ? 1.f : 0.f;
    const int last = ctx + tok0 + ntok - 1;            // the last key any row of the tile sees
    const int* table = block_table + (size_t)req * bt_stride;
    for (int k0 = split * LAT_KT; k0 <= last; k0 += splits * LAT_KT) {
        __syncthreads();
        const int nk = min(LAT_KT, last + 1 - k0);
        for (int i = threadIdx.x; i < nk * D; i += blockDim.x) {
            const int kk = i / D, d = i % D, pos = k0 + kk;
            const int page = table[pos / page_size];
            sk[kk * ldk + d] = to_float(plane[((size_t)page * page_size + pos % page_size) * D + d]);
        }
        __syncthreads();
        if (!row_ok || k0 > qpos) continue;
        // scores: lanes 0..KT-1 take one key each (the upper half of the wave idles here)
        float s = -INFINITY;
        if (lane < nk && k0 + lane <= qpos) {
            const float* kr = sk + lane * ldk;
            const float* qr = sq + wave * D;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qr[d], kr[d], dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
        const float fix = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * fix + wave_sum(p);
        m = m_new;
        __builtin_amdgcn_wave_barrier();                // (the wave's reads of the weights of the keys before are done)
        if (lane < LAT_KT) sp[wave * LAT_KT + lane] = p;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();                // a wave reads only what it wrote itself; its lanes run in step
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            if (c < cols) {
                const int col = c * TL_WAVE + lane;
                float a = acc[c] * fix;
                if (col < rank)
                    for (int kk = 0; kk < nk; ++kk) a = fmaf(sp[wave * LAT_KT + kk], sk[kk * ldk + col], a);
                acc[c] = a;
            }
        }
    }
    if (!row_ok) return;
    if (splits == 1) {
        const float inv = l > 0.f ? 1.f / l : 0.f;
        T* o = out + ((size_t)tok * heads + rh) * rank;
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const int col = c * TL_WAVE + lane;
            if (c < cols && col < rank) o[col] = from_float<T>(acc[c] * inv);
        }
    } else {
        const size_t prow = ((size_t)tok * heads + rh) * splits + split;
        float* o = part_o + prow * rank;
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const int col = c * TL_WAVE + lane;
            if (c < cols && col < rank) o[col] = acc[c];
        }
        if (lane == 0) { part_ml[prow * 2] = m; part_ml[prow * 2 + 1] = l; }
    }
}

// out[row] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s over the parts of a row, in the order of the parts.
template <typename T>
__global__ void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, T* __restrict__ out,
                                    int rows, int rank, int splits) {
    const int row = blockIdx.x;
    const float* ml = part_ml + (size_t)row * splits * 2;
    float M = -INFINITY;
    for (int s = 0; s < splits; ++s) M = fmaxf(M, ml[s * 2]);
    float den = 0.f;
    for (int s = 0; s < splits; ++s) den += (ml[s * 2] == -INFINITY) ? 0.f : expf(ml[s * 2] - M) * ml[s * 2 + 1];
    const float inv = den > 0.f ? 1.f / den : 0.f;
    for (int c = threadIdx.x; c < rank; c += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < splits; ++s)
            if (ml[s * 2] != -INFINITY) a = fmaf(expf(ml[s * 2] - M), part_o[((size_t)row * splits + s) * rank + c], a);
        out[(size_t)row * rank + c] = from_float<T>(a * inv);
    }
}

// q [tokens, q_ld]: per head rank + rot numbers (head h at column h * (rank + rot)); out [tokens, heads * rank];
// plane [pages, page_size, rank + rot]; sink float [heads] or null; tile_req null: tile i is the one token of request i.
extern "C" int tl_latent_attention(const void* q, int q_ld, void* out, const void* plane, const void* block_table, int bt_stride,
                                   const void* req_indptr, const void* ctx_lens, const void* tile_req, const void* tile_tok0,
                                   int num_tiles, int tokens, int tile_tokens, int heads, int rank, int rot, int page_size, float scale,
                                   const void* sink, int splits, void* part_o, void* part_ml, int dtype, hipStream_t stream) {
    TL_REQUIRE(num_tiles >= 0 && heads > 0 && rank > 0 && rot >= 0 && page_size > 0 && tile_tokens > 0, "latent_attention: bad sizes");
    TL_REQUIRE(rank <= 16 * TL_WAVE, "latent_attention: built for latents of up to %d numbers, got %d", 16 * TL_WAVE, rank);
    TL_REQUIRE(tile_tokens * min(heads, LAT_ROWS) <= LAT_ROWS, "latent_attention: a tile of %d tokens and %d heads has more than %d rows", tile_tokens, heads, LAT_ROWS);
    TL_REQUIRE(splits >= 1 && (splits == 1 || (part_o != nullptr && part_ml != nullptr)), "latent_attention: parts need their scratch");
    TL_REQUIRE(q_ld >= heads * (rank + rot), "latent_attention: query rows are too short");
    if (num_tiles == 0) return TL_OK;
    const int D = rank + rot;
    const size_t smem = sizeof(float) * ((size_t)LAT_KT * (D + 1) + (size_t)LAT_ROWS * D + LAT_ROWS * LAT_KT);
    TL_REQUIRE(smem <= 160 * 1024, "latent_attention: %zu bytes of shared memory for rows of %d numbers", smem, D);
    dim3 grid(num_tiles, (heads + LAT_ROWS - 1) / LAT_ROWS, splits), block(LAT_ROWS * TL_WAVE);
#define TL_ARGS(T) (const T*)q, q_ld, (T*)out, (const T*)plane, (const int*)block_table, bt_stride, (const int*)req_indptr, (const int*)ctx_lens, \
                   (const int*)tile_req, (const int*)tile_tok0, tile_tokens, heads, rank, rot, page_size, scale, (const float*)sink, splits,      \
                   (float*)part_o, (float*)part_ml
    if (dtype == TL_DT_F32) {
        auto kernel = latent_attention_kernel<float>;
        if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
            tl_set_error("latent_attention: cannot get %zu bytes of shared memory", smem); return TL_ERR_HIP;
        }
        kernel<<<grid, block, smem, stream>>>(TL_ARGS(float));
    } else if (dtype == TL_DT_BF16) {
        auto kernel = latent_attention_kernel<bf16_t>;
        if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
            tl_set_error("latent_attention: cannot get %zu bytes of shared memory", smem); return TL_ERR_HIP;
        }
        kernel<<<grid, block, smem, stream>>>(TL_ARGS(bf16_t));
    } else TL_REQUIRE(false, "latent_attention: unknown dtype %d", dtype);
#undef TL_ARGS
    TL_CHECK_LAUNCH("latent_attention");
    if (splits > 1) {
        const int rows = tokens * heads;
        if (dtype == TL_DT_F32) latent_merge_kernel<float><<<rows, 128, 0, stream>>>((const float*)part_o, (const float*)part_ml, (float*)out, rows, rank, splits);
        else latent_merge_kernel<bf16_t><<<rows, 128, 0, stream>>>((const float*)part_o, (const float*)part_ml, (bf16_t*)out, rows, rank, splits);
        TL_CHECK_LAUNCH("latent_merge");
    }
    return TL_OK;
}
