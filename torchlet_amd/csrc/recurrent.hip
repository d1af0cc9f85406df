// Recurrent mixers with a fixed-size state per request: the matrix-memory recurrence (mLSTM) and the
// gated per-head norm of its output.  State, gates, decays and the output's quotient are float whatever the
// activation type; queries, keys and values come in the activation type as the projection left them.
#include "common.h"

// A barrier that orders shared memory only: __syncthreads() also waits for every fetch from memory that is on its
// way (its fence covers global memory), which would end a prefetch at the first barrier after it.
__device__ __forceinline__ void shared_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ------------------------------------------------------------------ gates
__device__ __forceinline__ float soft_cap(float z, float cap) { return cap > 0.f ? cap * tanhf(z / cap) : z; }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// ------------------------------------------------------------------ the recurrence
// Per request and head a state of dim x vdim numbers S, dim numbers n and a running maximum m:
//   m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone;
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + denom_eps),        q scaled by qscale.
// n is one more column of S, the one whose "value" is 1 for every token: S'[:, n] = keep S[:, n] + take k, and n . q is
// that column's output.  A work-group owns COLS - 1 columns of one request's and head's S and a copy of the n column
// (so nothing is exchanged between work-groups; the first one stores n and m, and all of them read n and m from a
// copy taken before the launch, since a work-group may start after the first one has finished).  A lane owns one column and RPT rows of
// it, in registers for all tokens of the step: with COLS = 64 a wave holds RPT rows, with 32 or 16 it holds two or
// four groups of RPT rows side by side, which makes more and smaller work-groups where a step has few requests.
// Tokens are taken TB at a time: their q, k, v go to shared memory, one wave turns their gates into decays (the capped
// gates and the exponentials side by side, the running maximum one token after the other, as it is defined), every
// lane runs the TB updates of its rows and leaves its rows' shares of each token's sums, and the shares are added in the
// order of the rows.  A share is always that of four rows, whatever RPT and COLS are (a lane with RPT rows leaves RPT / 4
// of them), so a token's result does not depend on how the step was cut or on what else is in it: a prompt is run with
// few rows to a lane, because the time of a token is the chain of one lane's updates, a decode step with many rows and
// wide tiles, because its time is the stream of the states.
#define MLSTM_TB 16
#define MLSTM_SHARE 4

template <typename T, int RPT, int COLS>
__global__ void __launch_bounds__(1024)
mlstm_scan_kernel(const T* __restrict__ qkv, int ld, int k_off, int v_off,
                  const float* __restrict__ gates,          // [tokens, 2 * heads]: raw input gates, raw forget gates
                  float* __restrict__ state, size_t slot_stride, const int* __restrict__ slots, const float* __restrict__ before,
                  const int* __restrict__ req_indptr, float* __restrict__ out, int heads, int dim, int vdim,
                  float cap, float qscale, float denom_eps, int tb) {
    constexpr int RG = TL_WAVE / COLS;                 // groups of RPT rows a wave holds side by side
    extern __shared__ float smem[];
    const int waves = blockDim.x / TL_WAVE, wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    constexpr int SPL = RPT / MLSTM_SHARE;             // shares of a lane
    const int shares = waves * RG * SPL;               // >= ceil(dim / 4)
    // tb <= MLSTM_TB tokens are taken at a time: no more than the longest request of the step brings, so that a decode step's
    // work-groups need little shared memory and several fit a compute unit
    float* sq = smem;                                  // [tb][dim]
    float* sk = sq + tb * dim;                         // [tb][dim]
    float* sv = sk + tb * dim;                         // [tb][COLS]: the values of the tile's columns, 1 for the n column
    float* sd = sv + tb * COLS;                        // [tb][4]: keep, take, m after the token, (log input gate)
    float* part = sd + tb * 4;                         // [tb][shares][COLS]

    const int req = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * (COLS - 1);
    const int tok0 = req_indptr[req], tok1 = req_indptr[req + 1];
    if (tok0 >= tok1) return;
    const int c = lane % COLS, share = (wave * RG + lane / COLS) * SPL;     // the first of this lane's shares
    const bool is_n = c == COLS - 1;
    const int col = col0 + c;
    const bool col_ok = !is_n && col < vdim;
    const int row0 = share * MLSTM_SHARE;
    float* st = state + (size_t)slots[req] * slot_stride + (size_t)head * ((size_t)dim * vdim + dim + 1);
    float* st_n = st + (size_t)dim * vdim;
    const float* nm = before + ((size_t)req * heads + head) * (dim + 1);      // n and m as they were before the launch

    float S[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = row0 + r;
        S[r] = row < dim ? (is_n ? nm[row] : (col_ok ? st[(size_t)row * vdim + col] : 0.f)) : 0.f;
    }
    float m = nm[dim];                                 // (kept by the first wave, which turns the gates into decays)

    // A batch's q, k, v and raw gates are fetched into registers while the batch before is worked on (16-byte pieces of the
    // q and k rows where they are aligned), and go to shared memory, widened, when its sums have been read.
    constexpr int VEC = 16 / (int)sizeof(T);           // numbers of a 16-byte piece
    constexpr int QK_PF = (MLSTM_TB * 2 * RPT * RG + VEC * TL_WAVE - 1) / (VEC * TL_WAVE);     // pieces a thread fetches at most
    constexpr int V_PF = MLSTM_TB * COLS / TL_WAVE;    // values a thread fetches at most
    const bool vec_ok = dim % VEC == 0 && ld % VEC == 0 && k_off % VEC == 0 && ((uintptr_t)qkv % 16) == 0;
    const int dv = dim / VEC;
    uint4 qk_stage[QK_PF];
    T v_stage[V_PF];
    float g_stage[2] = {0.f, 0.f};
    auto fetch = [&](int base) {
        const int nb = min(tb, tok1 - base);
        if (vec_ok) {
#pragma unroll
            for (int j = 0; j < QK_PF; ++j) {
                const int idx = min((int)threadIdx.x + j * (int)blockDim.x, nb * 2 * dv - 1);       // (clamped: every lane fetches)
                const int t = idx / (2 * dv), rem = idx % (2 * dv);
                qk_stage[j] = *(const uint4*)(qkv + (size_t)(base + t) * ld + head * dim + (rem >= dv ? k_off : 0) + (rem % dv) * VEC);
            }
        }
#pragma unroll
        for (int j = 0; j < V_PF; ++j) {
            const int idx = min((int)threadIdx.x + j * (int)blockDim.x, nb * COLS - 1);
            const int vc = min(col0 + idx % COLS, vdim - 1);
            v_stage[j] = qkv[(size_t)(base + idx / COLS) * ld + v_off + head * vdim + vc];
        }
        if (wave == 0) {
            const float* g = gates + (size_t)(base + min(lane, nb - 1)) * 2 * heads;
            g_stage[0] = g[head];
            g_stage[1] = g[heads + head];
        }
    };
    fetch(tok0);
    for (int base = tok0; base < tok1; base += tb) {
        const int nb = min(tb, tok1 - base);
        shared_barrier();                               // the sums of the tokens before have been read
        if (vec_ok) {
#pragma unroll
            for (int j = 0; j < QK_PF; ++j) {
                const int idx = threadIdx.x + j * blockDim.x;
                if (idx < nb * 2 * dv) {
                    const int t = idx / (2 * dv), rem = idx % (2 * dv);
                    const bool is_k = rem >= dv;
                    float* dst = (is_k ? sk : sq) + t * dim + (rem % dv) * VEC;
                    const T* piece = (const T*)&qk_stage[j];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) dst[e] = is_k ? to_float(piece[e]) : to_float(piece[e]) * qscale;
                }
            }
        } else {
            for (int i = threadIdx.x; i < nb * dim; i += blockDim.x) {
                const int t = i / dim, d = i % dim;
                const T* row = qkv + (size_t)(base + t) * ld + head * dim;
                sq[t * dim + d] = to_float(row[d]) * qscale;
                sk[t * dim + d] = to_float(row[k_off + d]);
            }
        }
#pragma unroll
        for (int j = 0; j < V_PF; ++j) {
            const int idx = threadIdx.x + j * blockDim.x;
            if (idx < nb * COLS) {
                const int cc = idx % COLS;
                sv[idx] = cc == COLS - 1 ? 1.f : (col0 + cc < vdim ? to_float(v_stage[j]) : 0.f);
            }
        }
        if (wave == 0) {
            // the capped gates side by side, the running maximum token after token (every lane walks the same chain),
            // then the decays side by side
            const float gi = soft_cap(g_stage[0], cap), gf = log_sigmoid(soft_cap(g_stage[1], cap));
            float m_before = m, m_mine = m;
            for (int t = 0; t < nb; ++t) {             // (lane t's gates, read across the wave without a trip to shared memory)
                const float fi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gi), t));
                const float ff = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gf), t));
                const float m_new = fmaxf(ff + m, fi);
                if (lane == t) { m_before = m; m_mine = m_new; }
                m = m_new;
            }
            if (lane < nb) {
                sd[lane * 4] = expf(gf + m_before - m_mine);
                sd[lane * 4 + 1] = expf(gi - m_mine);
                sd[lane * 4 + 2] = m_mine;
            }
        }
        if (base + tb < tok1) fetch(base + tb);
        shared_barrier();
#pragma unroll 4
        for (int t = 0; t < nb; ++t) {
            const float keep = sd[t * 4], tv = sd[t * 4 + 1] * sv[t * COLS + c];
            const float* kt = sk + t * dim + row0;
            const float* qt = sq + t * dim + row0;
#pragma unroll
            for (int u = 0; u < SPL; ++u) {
                float o = 0.f;
#pragma unroll
                for (int r = MLSTM_SHARE * u; r < MLSTM_SHARE * (u + 1); ++r) {
                    if (row0 + r < dim) {
                        S[r] = fmaf(kt[r], tv, keep * S[r]);
                        o = fmaf(S[r], qt[r], o);
                    }
                }
                part[((size_t)t * shares + share + u) * COLS + c] = o;
            }
        }
        shared_barrier();
        for (int t = wave; t < nb; t += waves) {
            if (lane < COLS) {
                // the shares in four interleaved sums (shares 0, 4, 8, ...; 1, 5, 9, ...; ...), added up in their order:
                // one fixed order whatever the work-group's shape, and four chains of additions instead of one
                float o4[4] = {0.f, 0.f, 0.f, 0.f}, n4[4] = {0.f, 0.f, 0.f, 0.f};
                for (int w = 0; w < shares; w += 4) {          // (shares is a multiple of four or the tail is zeros of lanes without rows)
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (w + u < shares) {
                            const float* p = part + ((size_t)t * shares + w + u) * COLS;
                            o4[u] += p[lane];
                            n4[u] += p[COLS - 1];
                        }
                    }
                }
                const float osum = ((o4[0] + o4[1]) + o4[2]) + o4[3], nq = ((n4[0] + n4[1]) + n4[2]) + n4[3];
                if (lane < COLS - 1 && col0 + lane < vdim)
                    out[((size_t)(base + t) * heads + head) * vdim + col0 + lane] = osum / (fmaxf(fabsf(nq), expf(-sd[t * 4 + 2])) + denom_eps);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = row0 + r;
        if (row < dim) {
            if (col_ok) st[(size_t)row * vdim + col] = S[r];
            else if (is_n && blockIdx.x == 0) st_n[row] = S[r];
        }
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) st_n[dim] = m;
}

// n and m of the step's requests and heads, copied out of their slots: before[(req, head)] = [n (dim), m].
__global__ void mlstm_before_kernel(const float* __restrict__ state, size_t slot_stride, const int* __restrict__ slots,
                                    float* __restrict__ before, int heads, int dim, int vdim) {
    const int req = blockIdx.x / heads, head = blockIdx.x % heads;
    const float* src = state + (size_t)slots[req] * slot_stride + (size_t)head * ((size_t)dim * vdim + dim + 1) + (size_t)dim * vdim;
    float* dst = before + (size_t)blockIdx.x * (dim + 1);
    for (int i = threadIdx.x; i <= dim; i += blockDim.x) dst[i] = src[i];
}

template <typename T, int RPT, int COLS>
static int launch_mlstm_scan(const void* qkv, int ld, int k_off, int v_off, const void* gates, void* state, size_t slot_stride,
                             const void* slots, const void* before, const void* req_indptr, void* out, int requests, int heads, int dim, int vdim,
                             float cap, float qscale, float denom_eps, int tb, hipStream_t stream) {
    constexpr int RG = TL_WAVE / COLS;
    const int waves = (dim + RPT * RG - 1) / (RPT * RG);
    TL_REQUIRE(waves <= 16, "mlstm_scan: %d rows of a head do not fit a work-group of %d rows a lane and %d columns", dim, RPT, COLS);
    // tokens of a batch: as many as asked for, halved until their inputs and sums fit the shared memory (large heads)
    const size_t per_token = sizeof(float) * ((size_t)2 * dim + COLS + 4 + (size_t)waves * RG * (RPT / MLSTM_SHARE) * COLS);
    while (tb > 1 && per_token * tb > 144 * 1024) tb /= 2;
    const size_t smem = per_token * tb;
    TL_REQUIRE(smem <= 160 * 1024, "mlstm_scan: %zu bytes of shared memory for dim %d", smem, dim);
    auto kernel = mlstm_scan_kernel<T, RPT, COLS>;
    static size_t allowed = 48 * 1024;               // (per instance of the template)
    if (smem > allowed) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) { tl_set_error("mlstm_scan: cannot get %zu bytes of shared memory: %s", smem, hipGetErrorString(e)); return TL_ERR_HIP; }
        allowed = smem;
    }
    dim3 grid((vdim + COLS - 2) / (COLS - 1), heads, requests), block(waves * TL_WAVE);
    mlstm_before_kernel<<<requests * heads, 128, 0, stream>>>((const float*)state, slot_stride, (const int*)slots, (float*)before, heads, dim, vdim);
    TL_CHECK_LAUNCH("mlstm_before");
    kernel<<<grid, block, smem, stream>>>((const T*)qkv, ld, k_off, v_off, (const float*)gates, (float*)state, slot_stride,
                                           (const int*)slots, (const float*)before, (const int*)req_indptr, (float*)out, heads, dim, vdim, cap, qscale, denom_eps, tb);
    TL_CHECK_LAUNCH("mlstm_scan");
    return TL_OK;
}

static int tl_mlstm_units = 256;       // compute units the column tiles are dealt to
extern "C" void tl_mlstm_set_compute_units(int units) { if (units > 0) tl_mlstm_units = units; }

// qkv [tokens, ld]: queries at column 0 (heads * dim), keys at k_off, values at v_off (heads * vdim); gates float
// [tokens, 2 * heads]; state float [slots, heads, dim * vdim + dim + 1] with slot_stride floats between slots;
// out float [tokens, heads * vdim]; before: scratch of requests * heads * (dim + 1) floats.  Requests whose req_indptr range
// is empty are left alone.
extern "C" int tl_mlstm_scan(const void* qkv, int ld, int k_off, int v_off, const void* gates, void* state, long slot_stride,
                             const void* slots, const void* before, const void* req_indptr, void* out, int requests, int heads, int dim, int vdim,
                             float cap, float qscale, float denom_eps, int longest, int dtype, hipStream_t stream) {
    TL_REQUIRE(requests >= 0 && heads > 0 && dim > 0 && vdim > 0 && ld > 0, "mlstm_scan: bad sizes");
    const int tb = longest < 1 ? 1 : (longest < MLSTM_TB ? longest : MLSTM_TB);       // longest: the most tokens a request of the step brings
    TL_REQUIRE(dim <= 1024, "mlstm_scan: built for up to 1024 query/key dimensions per head, got %d", dim);
    TL_REQUIRE(slot_stride >= (long)heads * ((long)dim * vdim + dim + 1), "mlstm_scan: the state rows are too short");
    TL_REQUIRE(dtype == TL_DT_F32 || dtype == TL_DT_BF16, "mlstm_scan: unknown dtype %d", dtype);
    if (requests == 0) return TL_OK;
    // columns of a work-group: as few as it takes to give every compute unit one (the sums do not depend on the choice)
    const long heads_reqs = (long)heads * requests;
    const int cols = heads_reqs * ((vdim + 62) / 63) >= tl_mlstm_units ? 64 : heads_reqs * ((vdim + 30) / 31) >= tl_mlstm_units ? 32 : 16;
    // rows a lane keeps: as few as 16 waves of such lanes can hold the head's rows with, four at least
    const int need = (dim * cols + 16 * TL_WAVE - 1) / (16 * TL_WAVE);
    const int rpt = need <= 4 ? 4 : need <= 8 ? 8 : need <= 16 ? 16 : need <= 32 ? 32 : 64;
#define TL_MLSTM_C(R, C)                                                                                                       \
    return dtype == TL_DT_F32                                                                                                  \
        ? launch_mlstm_scan<float, R, C>(qkv, ld, k_off, v_off, gates, state, (size_t)slot_stride, slots, before, req_indptr, out,    \
                                         requests, heads, dim, vdim, cap, qscale, denom_eps, tb, stream)                      \
        : launch_mlstm_scan<bf16_t, R, C>(qkv, ld, k_off, v_off, gates, state, (size_t)slot_stride, slots, before, req_indptr, out,   \
                                          requests, heads, dim, vdim, cap, qscale, denom_eps, tb, stream)
#define TL_MLSTM(R)                                  \
    if (cols == 64) { TL_MLSTM_C(R, 64); }           \
    else if (cols == 32) { TL_MLSTM_C(R, 32); }      \
    else { TL_MLSTM_C(R, 16); }
    switch (rpt) {
        case 4: TL_MLSTM(4)
        case 8: TL_MLSTM(8)
        case 16: TL_MLSTM(16)
        case 32: TL_MLSTM(32)
        default: TL_MLSTM(64)
    }
#undef TL_MLSTM
#undef TL_MLSTM_C
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
