// Recurrent mixers with a fixed-size state per request: the matrix-memory recurrence (mLSTM), the gated delta rule behind its
// short convolutions, and the gated per-head norm of their outputs.  State, gates, decays and the output's quotient are float whatever the
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
// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * weight[h, :] * gate(g[t, h, :]) * gain; one wave per token and head.
// gate 0: sigmoid, 1: silu.  shared_weight: one vector of vdim numbers for all heads.  The rows of g and y may be longer than
// heads * vdim (views into wider buffers).  gate_first: the gate comes before the norm, y = u / sqrt(mean(u^2) + eps) * weight * gain
// with u = o * gate(g) (a "head" is then whatever stretch of the row is normed together).
template <typename T>
__global__ void gated_head_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate, int gate_ld,
                                       const void* __restrict__ weight, int weight_f32, int shared_weight, float eps,
                                       T* __restrict__ out, int out_ld, int rows, int heads, int vdim, int gate_kind, float gain, int gate_first) {
    const int row = blockIdx.x * (blockDim.x / TL_WAVE) + threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    if (row >= rows) return;
    const int t = row / heads, h = row % heads;
    const float* src = o + (size_t)row * vdim;
    const T* g = gate + (size_t)t * gate_ld + h * vdim;
    float ss = 0.f;
    for (int i = lane; i < vdim; i += TL_WAVE) {
        float u = src[i];
        if (gate_first) {
            const float z = to_float(g[i]);
            const float s = 1.f / (1.f + expf(-z));
            u *= gate_kind == 1 ? z * s : s;
        }
        ss = fmaf(u, u, ss);
    }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
    T* dst = out + (size_t)t * out_ld + h * vdim;
    const int w0 = shared_weight ? 0 : h * vdim;
    for (int i = lane; i < vdim; i += TL_WAVE) {
        const float z = to_float(g[i]);
        const float s = 1.f / (1.f + expf(-z));
        dst[i] = from_float<T>(src[i] * (gate_kind == 1 ? z * s : s) * inv * load_vec(weight, weight_f32, w0 + i) * gain);
    }
}

// The same for long stretches (more than 512 numbers normed together: all heads of a mixer as one): a work-group of 256 threads per token and
// stretch instead of a wave, the sum of squares joined through shared memory.
template <typename T>
__global__ void __launch_bounds__(256)
gated_row_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate, int gate_ld, const void* __restrict__ weight, int weight_f32,
                      int shared_weight, float eps, T* __restrict__ out, int out_ld, int heads, int vdim, int gate_kind, float gain, int gate_first) {
    __shared__ float red[16];
    const int row = blockIdx.x;
    const int t = row / heads, h = row % heads;
    const float* src = o + (size_t)row * vdim;
    const T* g = gate + (size_t)t * gate_ld + h * vdim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < vdim; i += blockDim.x) {
        float u = src[i];
        if (gate_first) {
            const float z = to_float(g[i]);
            const float s = 1.f / (1.f + expf(-z));
            u *= gate_kind == 1 ? z * s : s;
        }
        ss = fmaf(u, u, ss);
    }
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
    T* dst = out + (size_t)t * out_ld + h * vdim;
    const int w0 = shared_weight ? 0 : h * vdim;
    for (int i = threadIdx.x; i < vdim; i += blockDim.x) {
        const float z = to_float(g[i]);
        const float s = 1.f / (1.f + expf(-z));
        dst[i] = from_float<T>(src[i] * (gate_kind == 1 ? z * s : s) * inv * load_vec(weight, weight_f32, w0 + i) * gain);
    }
}

extern "C" int tl_gated_head_norm(const void* o, const void* gate, int gate_ld, const void* weight, int weight_f32, int shared_weight, float eps,
                                  void* out, int out_ld, int tokens, int heads, int vdim, int gate_kind, float gain, int gate_first, int dtype,
                                  hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && heads > 0 && vdim > 0 && gate_ld >= heads * vdim && out_ld >= heads * vdim, "gated_head_norm: bad sizes");
    TL_REQUIRE(gate_kind == 0 || gate_kind == 1, "gated_head_norm: unknown gate %d", gate_kind);
    if (tokens == 0) return TL_OK;
    const int rows = tokens * heads;
    if (vdim > 512) {
        if (dtype == TL_DT_F32)
            gated_row_norm_kernel<float><<<rows, 256, 0, stream>>>((const float*)o, (const float*)gate, gate_ld, weight, weight_f32, shared_weight, eps,
                                                                   (float*)out, out_ld, heads, vdim, gate_kind, gain, gate_first);
        else if (dtype == TL_DT_BF16)
            gated_row_norm_kernel<bf16_t><<<rows, 256, 0, stream>>>((const float*)o, (const bf16_t*)gate, gate_ld, weight, weight_f32, shared_weight, eps,
                                                                    (bf16_t*)out, out_ld, heads, vdim, gate_kind, gain, gate_first);
        else TL_REQUIRE(false, "gated_head_norm: unknown dtype %d", dtype);
        TL_CHECK_LAUNCH("gated_row_norm");
        return TL_OK;
    }
    dim3 grid((rows + 3) / 4), block(4 * TL_WAVE);
    if (dtype == TL_DT_F32)
        gated_head_norm_kernel<float><<<grid, block, 0, stream>>>((const float*)o, (const float*)gate, gate_ld, weight, weight_f32, shared_weight, eps,
                                                                  (float*)out, out_ld, rows, heads, vdim, gate_kind, gain, gate_first);
    else if (dtype == TL_DT_BF16)
        gated_head_norm_kernel<bf16_t><<<grid, block, 0, stream>>>((const float*)o, (const bf16_t*)gate, gate_ld, weight, weight_f32, shared_weight, eps,
                                                                   (bf16_t*)out, out_ld, rows, heads, vdim, gate_kind, gain, gate_first);
    else TL_REQUIRE(false, "gated_head_norm: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("gated_head_norm");
    return TL_OK;
}

// ------------------------------------------------------------------ gated delta rule: what the recurrence reads
// A token's convolved channels come in units: kv_heads query heads, kv_heads key heads (dim channels each), heads value heads (vdim
// channels each); one wave per token and unit.  Channel c at the request's i-th token of the step:
//   y = sum_j w[c][j] * x[i - (taps - 1) + j][c],   x[i'] = the projection of the step's token i' >= 0, else tail[taps - 1 + i'][c]
//   (the slot's last taps - 1 inputs from before the step, oldest first; zero for a new request), then silu;
//   query and key heads: y / sqrt(sum y^2 + unit_eps), queries times qscale.
// One more unit per token turns the raw gates into beta = sigmoid(b) and decay = exp(-exp(a_log) * softplus(a + dt_bias)).
#define DELTA_MAX_TAPS 8
#define DELTA_UNIT_MAX 4        // channels a lane holds: heads of up to 256 channels

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const T* __restrict__ proj, int ld, const float* __restrict__ conv_w, float* __restrict__ gates,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ state, size_t slot_stride,
                     size_t tail_off, const int* __restrict__ slots, const int* __restrict__ req_indptr, const int* __restrict__ token_req,
                     float* __restrict__ qkv, int heads, int kv_heads, int dim, int vdim, int taps, float qscale, float unit_eps) {
    const int t = blockIdx.x, lane = threadIdx.x % TL_WAVE;
    const int unit = blockIdx.y * (blockDim.x / TL_WAVE) + threadIdx.x / TL_WAVE;
    const int units = 2 * kv_heads + heads;
    if (unit > units) return;
    if (unit == units) {                               // the gates of the token's heads
        for (int h = lane; h < heads; h += TL_WAVE) {
            float* g = gates + (size_t)t * 2 * heads;
            const float b = g[h], a = g[heads + h];
            g[h] = 1.f / (1.f + expf(-b));
            g[heads + h] = expf(-expf(a_log[h]) * softplus_f(a + dt_bias[h]));
        }
        return;
    }
    const int C = 2 * kv_heads * dim + heads * vdim;
    const bool is_v = unit >= 2 * kv_heads;
    const int width = is_v ? vdim : dim;
    const int c0 = is_v ? 2 * kv_heads * dim + (unit - 2 * kv_heads) * vdim : unit * dim;
    const int req = token_req[t];
    const int i = t - req_indptr[req];                 // the token's place in its request's portion
    const float* tail = state + (size_t)slots[req] * slot_stride + tail_off;
    float y[DELTA_UNIT_MAX];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < DELTA_UNIT_MAX; ++u) {
        const int c = c0 + lane + u * TL_WAVE;
        y[u] = 0.f;
        if (lane + u * TL_WAVE < width) {
            float acc = 0.f;
            for (int j = 0; j < taps; ++j) {
                const int back = i - (taps - 1) + j;   // the input's place in the portion
                const float xv = back >= 0 ? to_float(proj[(size_t)(t - i + back) * ld + c]) : tail[(size_t)(taps - 1 + back) * C + c];
                acc = fmaf(conv_w[(size_t)c * taps + j], xv, acc);
            }
            y[u] = silu_f(acc);
            ss = fmaf(y[u], y[u], ss);
        }
    }
    float factor = 1.f;
    if (!is_v) {
        ss = wave_sum(ss);
        factor = 1.f / sqrtf(ss + unit_eps);
        if (unit < kv_heads) factor *= qscale;
    }
#pragma unroll
    for (int u = 0; u < DELTA_UNIT_MAX; ++u)
        if (lane + u * TL_WAVE < width) qkv[(size_t)t * C + c0 + lane + u * TL_WAVE] = y[u] * factor;
}

// After the step the tail of a request holds the last taps - 1 inputs of its channels: of the step's tokens, and before those of the
// old tail.  A thread owns a channel of a request and reads the old tail before it writes.
template <typename T>
__global__ void delta_tail_kernel(const T* __restrict__ proj, int ld, float* __restrict__ state, size_t slot_stride, size_t tail_off,
                                  const int* __restrict__ slots, const int* __restrict__ req_indptr, int C, int taps) {
    const int req = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    const int tok0 = req_indptr[req], n = req_indptr[req + 1] - tok0;
    if (c >= C || n <= 0) return;
    float* tail = state + (size_t)slots[req] * slot_stride + tail_off;
    float old[DELTA_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS - 1; ++j) old[j] = j < taps - 1 ? tail[(size_t)j * C + c] : 0.f;
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS - 1; ++j) {
        if (j < taps - 1) {
            const int back = n - (taps - 1) + j;       // place in the portion of what becomes entry j
            float v = 0.f;
            if (back >= 0) v = to_float(proj[(size_t)(tok0 + back) * ld + c]);
            else {
#pragma unroll
                for (int q = 0; q < DELTA_MAX_TAPS - 1; ++q)
                    if (q == j + n) v = old[q];
            }
            tail[(size_t)j * C + c] = v;
        }
    }
}

extern "C" int tl_delta_prepare(const void* proj, int ld, const void* conv_w, void* gates, const void* a_log, const void* dt_bias, void* state,
                                long slot_stride, long tail_off, const void* slots, const void* req_indptr, const void* token_req, void* qkv,
                                int tokens, int requests, int heads, int kv_heads, int dim, int vdim, int taps, float qscale, float unit_eps,
                                int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0, "delta_prepare: bad sizes");
    TL_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "delta_prepare: 1 to %d taps are built, not %d", DELTA_MAX_TAPS, taps);
    TL_REQUIRE(dim <= DELTA_UNIT_MAX * TL_WAVE && vdim <= DELTA_UNIT_MAX * TL_WAVE, "delta_prepare: heads of up to %d channels are built", DELTA_UNIT_MAX * TL_WAVE);
    const int C = 2 * kv_heads * dim + heads * vdim;
    TL_REQUIRE(ld >= C && tail_off >= 0 && slot_stride >= tail_off + (long)(taps - 1) * C, "delta_prepare: rows or state too short");
    TL_REQUIRE(dtype == TL_DT_F32 || dtype == TL_DT_BF16, "delta_prepare: unknown dtype %d", dtype);
    if (tokens == 0 || requests == 0) return TL_OK;
    const int units = 2 * kv_heads + heads + 1;
    dim3 grid(tokens, (units + 3) / 4), block(4 * TL_WAVE);
    dim3 tgrid((C + 255) / 256, requests), tblock(256);
    if (dtype == TL_DT_F32) {
        delta_prepare_kernel<float><<<grid, block, 0, stream>>>((const float*)proj, ld, (const float*)conv_w, (float*)gates, (const float*)a_log, (const float*)dt_bias,
            (const float*)state, (size_t)slot_stride, (size_t)tail_off, (const int*)slots, (const int*)req_indptr, (const int*)token_req, (float*)qkv,
            heads, kv_heads, dim, vdim, taps, qscale, unit_eps);
        TL_CHECK_LAUNCH("delta_prepare");
        if (taps > 1) delta_tail_kernel<float><<<tgrid, tblock, 0, stream>>>((const float*)proj, ld, (float*)state, (size_t)slot_stride, (size_t)tail_off,
                                                                             (const int*)slots, (const int*)req_indptr, C, taps);
    } else {
        delta_prepare_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)proj, ld, (const float*)conv_w, (float*)gates, (const float*)a_log, (const float*)dt_bias,
            (const float*)state, (size_t)slot_stride, (size_t)tail_off, (const int*)slots, (const int*)req_indptr, (const int*)token_req, (float*)qkv,
            heads, kv_heads, dim, vdim, taps, qscale, unit_eps);
        TL_CHECK_LAUNCH("delta_prepare");
        if (taps > 1) delta_tail_kernel<bf16_t><<<tgrid, tblock, 0, stream>>>((const bf16_t*)proj, ld, (float*)state, (size_t)slot_stride, (size_t)tail_off,
                                                                              (const int*)slots, (const int*)req_indptr, C, taps);
    }
    TL_CHECK_LAUNCH("delta_tail");
    return TL_OK;
}

// ------------------------------------------------------------------ gated delta rule: the recurrence
// Per request and head a state S of dim x vdim numbers; per token, with the decay g, the step size beta, unit q (scaled) and k:
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q.
// Column j of S needs only its own a_j = sum_r S[r][j] k[r] and b_j = sum_r S[r][j] q[r] (of the state before the decay) and k . q:
//   u_j = beta (v_j - g a_j);   o_j = g b_j + (k . q) u_j;   S[r][j] <- g S[r][j] + k[r] u_j.
// The 16 lanes of a row of the wave share a column: lane i of them owns the rows i RPL .. i RPL + RPL - 1 of it in registers for all
// tokens of the step (RPL = 4, 8, 12 or 16, fixed by dim alone), and they add their sums with four exchanges inside the row (pairs,
// quads, halves, the row: every lane gets the same bits).  The order of every sum is fixed by dim, so a token's result depends neither
// on how its request was cut into steps nor on what else the step holds.  A wave has 4 columns, a work-group of four waves 16.  The
// state of a head lies column by column ([vdim][dim]), so a lane's rows are side by side in memory and a wave fetches whole lines.
// Tokens are taken TB at a time (1, 4 or 16, by the longest portion of the step): their q, k, v, beta and g go to shared memory (the
// next batch is fetched into registers while this one is worked on) and every lane runs the TB updates of its rows; a request's last
// batch is filled up with tokens that change nothing (k = 0, beta = 0, decay 1), so the loop has no branch.
#define DELTA_L 16
#define DELTA_COLS 16           // columns of a work-group
#define DELTA_TB 16

template <int CTRL>
__device__ __forceinline__ float row_exchange(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// The sum of v over the 16 lanes of a row of the wave, in every one of them.
__device__ __forceinline__ float row16_sum(float v) {
    v += row_exchange<0xB1>(v);        // quad_perm [1, 0, 3, 2]: the neighbour
    v += row_exchange<0x4E>(v);        // quad_perm [2, 3, 0, 1]: the other pair of the quad
    v += row_exchange<0x141>(v);       // row_half_mirror: the other quad of the half
    v += row_exchange<0x140>(v);       // row_mirror: the other half
    return v;
}

// MODE 1: the delta rule.  MODE 0: the same recurrence without the correction, S <- g S + k v^T and o = S^T q, with one fixed decay per
// head (`head_decay`) in place of the tokens' gates: the decayed linear attention.  MODE 2: without the correction, with the tokens' own
// decays and step sizes, S <- g S + k (beta v)^T and o = S^T q + skip v with one skip factor per head (`head_decay` holds them): a
// selective state-space recurrence (k: the input matrix's row B, q: the output matrix's row C, beta: the step size, v: the input).
template <int RPL, int TB, int MODE>
__global__ void __launch_bounds__(256)
delta_scan_kernel(const float* __restrict__ qkv, const float* __restrict__ gates, const float* __restrict__ head_decay,
                  float* __restrict__ state, size_t slot_stride,
                  const int* __restrict__ slots, const int* __restrict__ req_indptr, float* __restrict__ out,
                  int heads, int kv_heads, int dim, int vdim) {
    constexpr int tb = TB;
    extern __shared__ float smem[];
    constexpr int ROWS = DELTA_L * RPL;                // >= dim
    float* sq = smem;                                  // [tb][ROWS]
    float* sk = sq + tb * ROWS;                        // [tb][ROWS]
    float* sv = sk + tb * ROWS;                        // [tb][DELTA_COLS]
    float* sg = sv + tb * DELTA_COLS;                  // [tb][2]: beta, decay
    const int req = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * DELTA_COLS;
    const int tok0 = req_indptr[req], tok1 = req_indptr[req + 1];
    if (tok0 >= tok1) return;
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    const int rg = lane & 15, cw = wave * 4 + (lane >> 4);       // the lane's group of rows and its column within the work-group
    const int col = col0 + cw, row0 = rg * RPL;
    const bool col_ok = col < vdim;
    const int C = 2 * kv_heads * dim + heads * vdim;
    const int qk_head = head / (heads / kv_heads);
    const int q_at = qk_head * dim, k_at = kv_heads * dim + qk_head * dim, v_at = 2 * kv_heads * dim + head * vdim + col0;
    float* st = state + (size_t)slots[req] * slot_stride + ((size_t)head * vdim + col) * dim + row0;

    float S[RPL];
    const bool whole = col_ok && row0 + RPL <= dim && (dim & 3) == 0 && ((uintptr_t)state & 15) == 0 && (slot_stride & 3) == 0;
    if (whole) {
#pragma unroll
        for (int r = 0; r < RPL; r += 4) {
            const float4 x = *(const float4*)(st + r);
            S[r] = x.x; S[r + 1] = x.y; S[r + 2] = x.z; S[r + 3] = x.w;
        }
    } else {
#pragma unroll
        for (int r = 0; r < RPL; ++r) S[r] = (col_ok && row0 + r < dim) ? st[r] : 0.f;
    }

    // a batch's numbers, fetched into registers one batch ahead: per token 2 * ROWS of q and k (zeros beyond dim), 16 of v, 2 gates
    constexpr int PER_TOKEN = 2 * ROWS + DELTA_COLS + 2;
    constexpr int STAGE = (TB * PER_TOKEN + 255) / 256;
    float stage[STAGE];
    auto fetch = [&](int base) {
        const int nb = min(tb, tok1 - base);
#pragma unroll
        for (int j = 0; j < STAGE; ++j) {
            const int idx = threadIdx.x + j * 256;
            float v = 0.f;
            if (idx < TB * PER_TOKEN) {
                const int t = idx / PER_TOKEN, e = idx % PER_TOKEN;
                if (t < nb) {
                    const float* row = qkv + (size_t)(base + t) * C;
                    if (e < ROWS) v = e < dim ? row[q_at + e] : 0.f;
                    else if (e < 2 * ROWS) v = e - ROWS < dim ? row[k_at + e - ROWS] : 0.f;
                    else if (e < 2 * ROWS + DELTA_COLS) v = col0 + e - 2 * ROWS < vdim ? row[v_at + e - 2 * ROWS] : 0.f;
                    else if (MODE != 0) v = gates[(size_t)(base + t) * 2 * heads + (e - 2 * ROWS - DELTA_COLS) * heads + head];
                    else v = e == PER_TOKEN - 1 ? head_decay[head] : 1.f;
                } else if (e == PER_TOKEN - 1) v = 1.f;        // beyond the request's last token: k = 0, beta = 0 and a decay of 1 leave the state as it is, to the bit
            }
            stage[j] = v;
        }
    };
    const float skip = MODE == 2 ? head_decay[head] : 0.f;
    fetch(tok0);
    for (int base = tok0; base < tok1; base += tb) {
        const int nb = min(tb, tok1 - base);
        __syncthreads();                               // the batch before has been worked on
#pragma unroll
        for (int j = 0; j < STAGE; ++j) {
            const int idx = threadIdx.x + j * 256;
            if (idx < TB * PER_TOKEN) {
                const int t = idx / PER_TOKEN, e = idx % PER_TOKEN;
                if (e < ROWS) sq[t * ROWS + e] = stage[j];
                else if (e < 2 * ROWS) sk[t * ROWS + e - ROWS] = stage[j];
                else if (e < 2 * ROWS + DELTA_COLS) sv[t * DELTA_COLS + e - 2 * ROWS] = stage[j];
                else sg[t * 2 + e - 2 * ROWS - DELTA_COLS] = stage[j];
            }
        }
        if (base + tb < tok1) fetch(base + tb);
        __syncthreads();
        // the batch's tokens one after the other, the loop written out without a branch (a batch is always whole: see above): nothing
        // in it writes memory, so the fetches of the tokens to come move ahead of the sums of the token at hand; the outputs wait in
        // registers for the end of the batch
        float obuf[TB];
#pragma unroll
        for (int t = 0; t < TB; ++t) {
            {
                const float* kt = sk + t * ROWS + row0;
                const float* qt = sq + t * ROWS + row0;
                float kr[RPL], qr[RPL];
#pragma unroll
                for (int r = 0; r < RPL; r += 4) {
                    const float4 k4 = *(const float4*)(kt + r), q4 = *(const float4*)(qt + r);
                    kr[r] = k4.x; kr[r + 1] = k4.y; kr[r + 2] = k4.z; kr[r + 3] = k4.w;
                    qr[r] = q4.x; qr[r + 1] = q4.y; qr[r + 2] = q4.z; qr[r + 3] = q4.w;
                }
                const float beta = sg[t * 2], g = sg[t * 2 + 1], vt = sv[t * DELTA_COLS + cw];
                // four chains of additions each, joined in a fixed order
                float a4[4] = {0.f, 0.f, 0.f, 0.f}, b4[4] = {0.f, 0.f, 0.f, 0.f}, c4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int r = 0; r < RPL; ++r) {
                    if (MODE == 1) a4[r & 3] = fmaf(S[r], kr[r], a4[r & 3]);
                    b4[r & 3] = fmaf(S[r], qr[r], b4[r & 3]);
                    c4[r & 3] = fmaf(kr[r], qr[r], c4[r & 3]);
                }
                const float a = MODE == 1 ? row16_sum((a4[0] + a4[1]) + (a4[2] + a4[3])) : 0.f;
                const float b = row16_sum((b4[0] + b4[1]) + (b4[2] + b4[3]));
                const float kq = row16_sum((c4[0] + c4[1]) + (c4[2] + c4[3]));
                const float u = MODE == 1 ? beta * (vt - g * a) : (MODE == 2 ? beta * vt : vt);
#pragma unroll
                for (int r = 0; r < RPL; ++r) S[r] = fmaf(kr[r], u, g * S[r]);
                obuf[t] = MODE == 2 ? fmaf(skip, vt, fmaf(kq, u, g * b)) : fmaf(kq, u, g * b);
            }
        }
        if (rg == 0 && col_ok) {
            float* orow = out + ((size_t)base * heads + head) * vdim + col;
#pragma unroll
            for (int t = 0; t < TB; ++t)
                if (t < nb) orow[(size_t)t * heads * vdim] = obuf[t];
        }
    }
    if (whole) {
#pragma unroll
        for (int r = 0; r < RPL; r += 4) *(float4*)(st + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
    } else if (col_ok) {
#pragma unroll
        for (int r = 0; r < RPL; ++r)
            if (row0 + r < dim) st[r] = S[r];
    }
}

// state: per slot, from its start, heads x [vdim][dim] floats (a head's state column by column).
template <int MODE>
static int launch_delta_scan(const void* qkv, const void* gates, const void* head_decay, void* state, long slot_stride, const void* slots,
                             const void* req_indptr, void* out, int requests, int heads, int kv_heads, int dim, int vdim, int longest, hipStream_t stream) {
    const int rpl = dim <= 64 ? 4 : dim <= 128 ? 8 : dim <= 192 ? 12 : 16;
    // tokens of a batch: 1 for a step of single tokens, 4 for short portions, else 16 (a batch is always worked through whole)
    const int tb = longest <= 1 ? 1 : (longest <= 4 ? 4 : DELTA_TB);
    const size_t smem = sizeof(float) * (size_t)tb * (2 * DELTA_L * rpl + DELTA_COLS + 2);
    dim3 grid((vdim + DELTA_COLS - 1) / DELTA_COLS, heads, requests), block(256);
#define TL_DELTA_B(R, B)                                                                                                                   \
    delta_scan_kernel<R, B, MODE><<<grid, block, smem, stream>>>((const float*)qkv, (const float*)gates, (const float*)head_decay, (float*)state, \
                                                           (size_t)slot_stride, (const int*)slots, (const int*)req_indptr, (float*)out, heads, kv_heads, dim, vdim)
#define TL_DELTA(R)                        \
    if (tb == 1) TL_DELTA_B(R, 1);         \
    else if (tb == 4) TL_DELTA_B(R, 4);    \
    else TL_DELTA_B(R, DELTA_TB)
    if (rpl == 4) { TL_DELTA(4); }
    else if (rpl == 8) { TL_DELTA(8); }
    else if (rpl == 12) { TL_DELTA(12); }
    else { TL_DELTA(16); }
#undef TL_DELTA
#undef TL_DELTA_B
    return TL_OK;
}

extern "C" int tl_delta_scan(const void* qkv, const void* gates, void* state, long slot_stride, const void* slots, const void* req_indptr,
                             void* out, int requests, int heads, int kv_heads, int dim, int vdim, int longest, hipStream_t stream) {
    TL_REQUIRE(requests >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0, "delta_scan: bad sizes");
    TL_REQUIRE(dim <= DELTA_L * 16, "delta_scan: built for up to %d query/key dimensions per head, got %d", DELTA_L * 16, dim);
    TL_REQUIRE(slot_stride >= (long)heads * dim * vdim, "delta_scan: the state rows are too short");
    TL_REQUIRE(requests <= 65535 && heads <= 65535, "delta_scan: too many requests or heads for one launch");
    if (requests == 0) return TL_OK;
    launch_delta_scan<1>(qkv, gates, nullptr, state, slot_stride, slots, req_indptr, out, requests, heads, kv_heads, dim, vdim, longest, stream);
    TL_CHECK_LAUNCH("delta_scan");
    return TL_OK;
}

// ------------------------------------------------------------------ decayed linear attention
// Per head S <- decay[head] S + k v^T, o = S^T q over the step's tokens, request by request from the state its slot holds: qkv float
// [T, 2 * heads * dim + heads * vdim] (queries, keys, values, head by head), state as the delta rule's, out float [T, heads * vdim].
extern "C" int tl_decay_scan(const void* qkv, const void* decay, void* state, long slot_stride, const void* slots, const void* req_indptr,
                             void* out, int requests, int heads, int dim, int vdim, int longest, hipStream_t stream) {
    TL_REQUIRE(requests >= 0 && heads > 0 && dim > 0 && vdim > 0 && decay, "decay_scan: bad sizes");
    TL_REQUIRE(dim <= DELTA_L * 16, "decay_scan: built for up to %d query/key dimensions per head, got %d", DELTA_L * 16, dim);
    TL_REQUIRE(slot_stride >= (long)heads * dim * vdim, "decay_scan: the state rows are too short");
    TL_REQUIRE(requests <= 65535 && heads <= 65535, "decay_scan: too many requests or heads for one launch");
    if (requests == 0) return TL_OK;
    launch_delta_scan<0>(qkv, nullptr, decay, state, slot_stride, slots, req_indptr, out, requests, heads, heads, dim, vdim, longest, stream);
    TL_CHECK_LAUNCH("decay_scan");
    return TL_OK;
}

// ------------------------------------------------------------------ selective state-space recurrence (Mamba-2)
// Per head S <- decay S + dt B x^T (S: state x vdim), y = S^T C + D x, with B and C shared by the heads of a group.  qkv float [T, 2 * groups *
// state + heads * vdim] as selective_prepare leaves it (C, B, x), gates float [T, 2 * heads] (dt, decay), skip float [heads] (D); the
// state as the delta rule's ([vdim][state] per head), out float [T, heads * vdim].
extern "C" int tl_selective_scan(const void* qkv, const void* gates, const void* skip, void* state, long slot_stride, const void* slots,
                                 const void* req_indptr, void* out, int requests, int heads, int groups, int dim, int vdim, int longest, hipStream_t stream) {
    TL_REQUIRE(requests >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && dim > 0 && vdim > 0 && gates && skip, "selective_scan: bad sizes");
    TL_REQUIRE(dim <= DELTA_L * 16, "selective_scan: built for states of up to %d numbers per column, got %d", DELTA_L * 16, dim);
    TL_REQUIRE(slot_stride >= (long)heads * dim * vdim, "selective_scan: the state rows are too short");
    TL_REQUIRE(requests <= 65535 && heads <= 65535, "selective_scan: too many requests or heads for one launch");
    if (requests == 0) return TL_OK;
    launch_delta_scan<2>(qkv, gates, skip, state, slot_stride, slots, req_indptr, out, requests, heads, groups, dim, vdim, longest, stream);
    TL_CHECK_LAUNCH("selective_scan");
    return TL_OK;
}

// What that recurrence reads, made from the projection of the step's tokens.  proj [T, ld] holds per token, from column x_off on, the
// `channels` = inner + 2 * groups * state convolved channels [x | B | C] and after them `heads` raw step sizes.  Channel c at the request's
// i-th token of the step: y = silu(bias[c] + sum_j w[c][j] * in[i - (taps - 1) + j][c]) with in[i'] the projection of the step's token
// i' >= 0, else tail[taps - 1 + i'][c] (the slot's last taps - 1 inputs from before the step; zero for a new request).  y goes to qkv
// float [T, channels] in the order the recurrence reads: C, B, x.  gates float [T, 2 * heads] receives dt = softplus(raw + dt_bias) and
// decay = exp(-exp(a_log) * dt).  One thread per token and channel (or head).
template <typename T>
__global__ void __launch_bounds__(256)
selective_prepare_kernel(const T* __restrict__ proj, int ld, int x_off, const float* __restrict__ conv_w, const float* __restrict__ conv_b,
                         float* __restrict__ gates, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                         const float* __restrict__ state, size_t slot_stride, size_t tail_off, const int* __restrict__ slots,
                         const int* __restrict__ req_indptr, const int* __restrict__ token_req, float* __restrict__ qkv, int heads, int inner,
                         int gn, int taps) {
    const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    const int channels = inner + 2 * gn;
    if (c >= channels + heads) return;
    const T* row = proj + (size_t)t * ld + x_off;
    if (c >= channels) {
        const int h = c - channels;
        const float dt = softplus_f(to_float(row[c]) + dt_bias[h]);
        gates[(size_t)t * 2 * heads + h] = dt;
        gates[(size_t)t * 2 * heads + heads + h] = expf(-expf(a_log[h]) * dt);
        return;
    }
    const int req = token_req[t];
    const int i = t - req_indptr[req];
    const float* tail = state + (size_t)slots[req] * slot_stride + tail_off;
    float acc = conv_b[c];
    for (int j = 0; j < taps; ++j) {
        const int back = i - (taps - 1) + j;
        const float xv = back >= 0 ? to_float(proj[(size_t)(t - i + back) * ld + x_off + c]) : tail[(size_t)(taps - 1 + back) * channels + c];
        acc = fmaf(conv_w[(size_t)c * taps + j], xv, acc);
    }
    const int to = c < inner ? 2 * gn + c : (c < inner + gn ? gn + (c - inner) : c - inner - gn);
    qkv[(size_t)t * channels + to] = silu_f(acc);
}

extern "C" int tl_selective_prepare(const void* proj, int ld, int x_off, const void* conv_w, const void* conv_b, void* gates, const void* a_log,
                                    const void* dt_bias, void* state, long slot_stride, long tail_off, const void* slots, const void* req_indptr,
                                    const void* token_req, void* qkv, int tokens, int requests, int heads, int inner, int gn, int taps, int dtype,
                                    hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && inner > 0 && gn > 0 && x_off >= 0, "selective_prepare: bad sizes");
    TL_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "selective_prepare: 1 to %d taps are built, not %d", DELTA_MAX_TAPS, taps);
    const int channels = inner + 2 * gn;
    TL_REQUIRE(ld >= x_off + channels + heads && tail_off >= 0 && slot_stride >= tail_off + (long)(taps - 1) * channels, "selective_prepare: rows or state too short");
    TL_REQUIRE(dtype == TL_DT_F32 || dtype == TL_DT_BF16, "selective_prepare: unknown dtype %d", dtype);
    TL_REQUIRE(requests <= 65535 && (channels + heads + 255) / 256 <= 65535, "selective_prepare: too many requests or channels for one launch");
    if (tokens == 0 || requests == 0) return TL_OK;
    dim3 grid(tokens, (channels + heads + 255) / 256), block(256);
    dim3 tgrid((channels + 255) / 256, requests), tblock(256);
#define TL_SP(T)                                                                                                                                  \
    selective_prepare_kernel<T><<<grid, block, 0, stream>>>((const T*)proj, ld, x_off, (const float*)conv_w, (const float*)conv_b, (float*)gates,     \
        (const float*)a_log, (const float*)dt_bias, (const float*)state, (size_t)slot_stride, (size_t)tail_off, (const int*)slots,               \
        (const int*)req_indptr, (const int*)token_req, (float*)qkv, heads, inner, gn, taps);                                                      \
    TL_CHECK_LAUNCH("selective_prepare");                                                                                                         \
    if (taps > 1) delta_tail_kernel<T><<<tgrid, tblock, 0, stream>>>((const T*)proj + x_off, ld, (float*)state, (size_t)slot_stride, (size_t)tail_off, \
                                                                     (const int*)slots, (const int*)req_indptr, channels, taps)
    if (dtype == TL_DT_F32) { TL_SP(float); } else { TL_SP(bf16_t); }
#undef TL_SP
    TL_CHECK_LAUNCH("selective_tail");
    return TL_OK;
}

// out[t, c] = silu(float(x[t, c])) for the first `cols` columns of every row (the rows of x may be longer).
template <typename T>
__global__ void silu_float_kernel(const T* __restrict__ x, int ld, float* __restrict__ out, int cols, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const float v = to_float(x[(i / cols) * ld + i % cols]);
    out[i] = v / (1.f + expf(-v));
}

extern "C" int tl_silu_float(const void* x, int ld, void* out, int rows, int cols, int dtype, hipStream_t stream) {
    TL_REQUIRE(rows >= 0 && cols > 0 && ld >= cols, "silu_float: bad sizes");
    if (rows == 0) return TL_OK;
    const size_t total = (size_t)rows * cols;
    const int grid = (int)((total + 255) / 256);
    if (dtype == TL_DT_F32) silu_float_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ld, (float*)out, cols, total);
    else if (dtype == TL_DT_BF16) silu_float_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ld, (float*)out, cols, total);
    else TL_REQUIRE(false, "silu_float: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("silu_float");
    return TL_OK;
}
