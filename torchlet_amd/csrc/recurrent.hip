// Recurrent mixers with a fixed-size state per request: the matrix-memory recurrence (mLSTM) and the
// gated per-head norm of its output.  State, gates, decays and the output's quotient are float whatever the
// activation type; queries, keys and values come in the activation type as the projection left them.
#include "common.h"

// ------------------------------------------------------------------ gates
__device__ __forceinline__ float soft_cap(float z, float cap) { return cap > 0.f ? cap * tanhf(z / cap) : z; }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// ------------------------------------------------------------------ the recurrence
// Per request and head a state of dim x vdim numbers S, dim numbers n and a running maximum m:
//   m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone;
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + denom_eps),        q scaled by qscale.
// A work-group owns the columns [64 * blockIdx.x, +64) of one request's and head's S: a lane owns one
// column, a wave the RPT rows [wave * RPT, +RPT) of it, in registers for all tokens of the step.  Every
// work-group of a head keeps n and m for itself (they are cheap); the one of the first columns stores them.
// Tokens are taken TB at a time: their q, k, v and gates go to shared memory, every wave runs the TB updates
// of its rows and leaves its part of each token's sums over the rows, and the parts are added in the order of
// the waves, so a token's result does not depend on how the step was cut.
#define MLSTM_TB 8
#define MLSTM_COLS 64

template <typename T, int RPT>
__global__ void __launch_bounds__(1024)
mlstm_scan_kernel(const T* __restrict__ qkv, int ld, int k_off, int v_off,
                  const float* __restrict__ gates,          // [tokens, 2 * heads]: raw input gates, raw forget gates
                  float* __restrict__ state, size_t slot_stride, const int* __restrict__ slots,
                  const int* __restrict__ req_indptr, float* __restrict__ out, int heads, int dim, int vdim,
                  float cap, float qscale, float denom_eps) {
    extern __shared__ float smem[];
    const int waves = blockDim.x / TL_WAVE, wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    float* sq = smem;                                  // [TB][dim]
    float* sk = sq + MLSTM_TB * dim;                   // [TB][dim]
    float* sv = sk + MLSTM_TB * dim;                   // [TB][64]
    float* sg = sv + MLSTM_TB * MLSTM_COLS;            // [TB][2]: log input gate, log forget gate
    float* sm = sg + MLSTM_TB * 2;                     // [TB]: the running maximum after each token
    float* part = sm + MLSTM_TB;                       // [TB][waves][65]: a wave's share of o (64 columns) and of n.q

    const int req = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * MLSTM_COLS;
    const int tok0 = req_indptr[req], tok1 = req_indptr[req + 1];
    if (tok0 >= tok1) return;
    const int col = col0 + lane;
    const bool col_ok = col < vdim;
    const int row0 = wave * RPT;
    float* st = state + (size_t)slots[req] * slot_stride + (size_t)head * ((size_t)dim * vdim + dim + 1);
    float* st_n = st + (size_t)dim * vdim;

    float S[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) S[r] = (col_ok && row0 + r < dim) ? st[(size_t)(row0 + r) * vdim + col] : 0.f;
    const bool n_ok = lane < RPT && row0 + lane < dim;      // lane r of a wave keeps n of the wave's row r
    float n = n_ok ? st_n[row0 + lane] : 0.f;
    float m = st_n[dim];

    for (int base = tok0; base < tok1; base += MLSTM_TB) {
        const int nb = min(MLSTM_TB, tok1 - base);
        __syncthreads();                               // the sums of the tokens before have been read
        for (int i = threadIdx.x; i < nb * dim; i += blockDim.x) {
            const int t = i / dim, d = i % dim;
            const T* row = qkv + (size_t)(base + t) * ld + head * dim;
            sq[t * dim + d] = to_float(row[d]) * qscale;
            sk[t * dim + d] = to_float(row[k_off + d]);
        }
        for (int i = threadIdx.x; i < nb * MLSTM_COLS; i += blockDim.x) {
            const int t = i / MLSTM_COLS, c = col0 + i % MLSTM_COLS;
            sv[i] = c < vdim ? to_float(qkv[(size_t)(base + t) * ld + v_off + head * vdim + c]) : 0.f;
        }
        if (threadIdx.x < nb) {
            const float* g = gates + (size_t)(base + threadIdx.x) * 2 * heads;
            sg[threadIdx.x * 2] = soft_cap(g[head], cap);
            sg[threadIdx.x * 2 + 1] = log_sigmoid(soft_cap(g[heads + head], cap));
        }
        __syncthreads();
        for (int t = 0; t < nb; ++t) {
            const float gi = sg[t * 2], gf = sg[t * 2 + 1];
            const float m_new = fmaxf(gf + m, gi);
            const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
            m = m_new;
            const float tv = take * sv[t * MLSTM_COLS + lane];
            const float* kt = sk + t * dim + row0;
            const float* qt = sq + t * dim + row0;
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < RPT; ++r) {
                if (row0 + r < dim) {
                    S[r] = fmaf(kt[r], tv, keep * S[r]);
                    o = fmaf(S[r], qt[r], o);
                }
            }
            float nq = 0.f;
            if (n_ok) {
                n = fmaf(take, kt[lane], keep * n);
                nq = n * qt[lane];
            }
            nq = wave_sum(nq);
            float* p = part + ((size_t)t * waves + wave) * (MLSTM_COLS + 1);
            p[lane] = o;
            if (lane == 0) p[MLSTM_COLS] = nq;
            if (threadIdx.x == 0) sm[t] = m;
        }
        __syncthreads();
        for (int t = wave; t < nb; t += waves) {
            float osum = 0.f, nq = 0.f;
            for (int w = 0; w < waves; ++w) {
                const float* p = part + ((size_t)t * waves + w) * (MLSTM_COLS + 1);
                osum += p[lane];
                nq += p[MLSTM_COLS];
            }
            if (col_ok)
                out[((size_t)(base + t) * heads + head) * vdim + col] = osum / (fmaxf(fabsf(nq), expf(-sm[t])) + denom_eps);
        }
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r)
        if (col_ok && row0 + r < dim) st[(size_t)(row0 + r) * vdim + col] = S[r];
    if (blockIdx.x == 0) {
        if (n_ok) st_n[row0 + lane] = n;
        if (threadIdx.x == 0) st_n[dim] = m;
    }
}

template <typename T, int RPT>
static int launch_mlstm_scan(const void* qkv, int ld, int k_off, int v_off, const void* gates, void* state, size_t slot_stride,
                             const void* slots, const void* req_indptr, void* out, int requests, int heads, int dim, int vdim,
                             float cap, float qscale, float denom_eps, hipStream_t stream) {
    const int waves = (dim + RPT - 1) / RPT;
    const size_t smem = sizeof(float) * ((size_t)2 * MLSTM_TB * dim + MLSTM_TB * MLSTM_COLS + 3 * MLSTM_TB +
                                         (size_t)MLSTM_TB * waves * (MLSTM_COLS + 1));
    TL_REQUIRE(smem <= 160 * 1024, "mlstm_scan: %zu bytes of shared memory for dim %d", smem, dim);
    auto kernel = mlstm_scan_kernel<T, RPT>;
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) { tl_set_error("mlstm_scan: cannot get %zu bytes of shared memory: %s", smem, hipGetErrorString(e)); return TL_ERR_HIP; }
    }
    dim3 grid((vdim + MLSTM_COLS - 1) / MLSTM_COLS, heads, requests), block(waves * TL_WAVE);
    kernel<<<grid, block, smem, stream>>>((const T*)qkv, ld, k_off, v_off, (const float*)gates, (float*)state, slot_stride,
                                           (const int*)slots, (const int*)req_indptr, (float*)out, heads, dim, vdim, cap, qscale, denom_eps);
    TL_CHECK_LAUNCH("mlstm_scan");
    return TL_OK;
}

// qkv [tokens, ld]: queries at column 0 (heads * dim), keys at k_off, values at v_off (heads * vdim); gates float
// [tokens, 2 * heads]; state float [slots, heads, dim * vdim + dim + 1] with slot_stride floats between slots;
// out float [tokens, heads * vdim].  Requests whose req_indptr range is empty are left alone.
extern "C" int tl_mlstm_scan(const void* qkv, int ld, int k_off, int v_off, const void* gates, void* state, long slot_stride,
                             const void* slots, const void* req_indptr, void* out, int requests, int heads, int dim, int vdim,
                             float cap, float qscale, float denom_eps, int dtype, hipStream_t stream) {
    TL_REQUIRE(requests >= 0 && heads > 0 && dim > 0 && vdim > 0 && ld > 0, "mlstm_scan: bad sizes");
    TL_REQUIRE(dim <= 1024, "mlstm_scan: built for up to 1024 query/key dimensions per head, got %d", dim);
    TL_REQUIRE(slot_stride >= (long)heads * ((long)dim * vdim + dim + 1), "mlstm_scan: the state rows are too short");
    if (requests == 0) return TL_OK;
    // rows a thread keeps: few for small heads (more waves at work), at most 16 waves to a work-group
    const int rpt = dim <= 64 ? 4 : dim <= 128 ? 8 : dim <= 256 ? 16 : dim <= 512 ? 32 : 64;
#define TL_MLSTM(R)                                                                                                            \
    return dtype == TL_DT_F32                                                                                                  \
        ? launch_mlstm_scan<float, R>(qkv, ld, k_off, v_off, gates, state, (size_t)slot_stride, slots, req_indptr, out,       \
                                      requests, heads, dim, vdim, cap, qscale, denom_eps, stream)                             \
        : launch_mlstm_scan<bf16_t, R>(qkv, ld, k_off, v_off, gates, state, (size_t)slot_stride, slots, req_indptr, out,      \
                                       requests, heads, dim, vdim, cap, qscale, denom_eps, stream)
    TL_REQUIRE(dtype == TL_DT_F32 || dtype == TL_DT_BF16, "mlstm_scan: unknown dtype %d", dtype);
    switch (rpt) {
        case 4: TL_MLSTM(4);
        case 8: TL_MLSTM(8);
        case 16: TL_MLSTM(16);
        case 32: TL_MLSTM(32);
        default: TL_MLSTM(64);
    }
#undef TL_MLSTM
}

// ------------------------------------------------------------------ gated per-head norm
// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * weight[h, :] * sigmoid(gate[t, h, :]); one wave per token and head.
template <typename T>
__global__ void gated_head_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate, int gate_ld,
                                       const void* __restrict__ weight, int weight_f32, float eps,
                                       T* __restrict__ out, int rows, int heads, int vdim) {
    const int row = blockIdx.x * (blockDim.x / TL_WAVE) + threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    if (row >= rows) return;
    const int t = row / heads, h = row % heads;
    const float* src = o + (size_t)row * vdim;
    float ss = 0.f;
    for (int i = lane; i < vdim; i += TL_WAVE) ss = fmaf(src[i], src[i], ss);
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
    const T* g = gate + (size_t)t * gate_ld + h * vdim;
    T* dst = out + (size_t)row * vdim;
    for (int i = lane; i < vdim; i += TL_WAVE) {
        const float z = to_float(g[i]);
        dst[i] = from_float<T>(src[i] * inv * load_vec(weight, weight_f32, h * vdim + i) * (1.f / (1.f + expf(-z))));
    }
}

extern "C" int tl_gated_head_norm(const void* o, const void* gate, int gate_ld, const void* weight, int weight_f32, float eps,
                                  void* out, int tokens, int heads, int vdim, int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && heads > 0 && vdim > 0 && gate_ld >= heads * vdim, "gated_head_norm: bad sizes");
    if (tokens == 0) return TL_OK;
    const int rows = tokens * heads;
    dim3 grid((rows + 3) / 4), block(4 * TL_WAVE);
    if (dtype == TL_DT_F32)
        gated_head_norm_kernel<float><<<grid, block, 0, stream>>>((const float*)o, (const float*)gate, gate_ld, weight, weight_f32, eps, (float*)out, rows, heads, vdim);
    else if (dtype == TL_DT_BF16)
        gated_head_norm_kernel<bf16_t><<<grid, block, 0, stream>>>((const float*)o, (const bf16_t*)gate, gate_ld, weight, weight_f32, eps, (bf16_t*)out, rows, heads, vdim);
    else TL_REQUIRE(false, "gated_head_norm: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("gated_head_norm");
    return TL_OK;
}
