// Matrix products over groups (one weight matrix per group: an expert and the tokens routed to it, or a head and
// its slice of every token's row), the router's choice of experts, the sort of tokens by expert, the weighted sum
// of the chosen experts' outputs, and the elementwise activation of a dense feed-forward.  Sums are float.
#include "common.h"

#define ACT_NONE 0
#define ACT_RELU2 1
#define ACT_SILU 2
#define ACT_GELU_TANH 3
#define ACT_GELU 4        // the exact form, with the error function
#define ACT_PAIRS 16      // added to one of the above: the product's columns 2i and 2i + 1 are a gate and an up value, the output act(gate) * up

__device__ __forceinline__ float activate(float v, int act) {
    if (act == ACT_RELU2) { v = fmaxf(v, 0.f); return v * v; }
    if (act == ACT_SILU) return v / (1.f + expf(-v));
    if (act == ACT_GELU_TANH) return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    if (act == ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.7071067811865476f));
    return v;
}

__host__ __device__ __forceinline__ bool known_activation(int act) { return (act & ~ACT_PAIRS) >= ACT_NONE && (act & ~ACT_PAIRS) <= ACT_GELU; }

// ------------------------------------------------------------------ grouped product
// out[row(m), g_out + n] = act(sum_k a[src(m), g_a + k] * w[g][n][k]) for the rows m of group g, in tiles of 64 x 64
// with K in steps of 16 through shared memory; a thread owns a 4 x 4 block of the tile.  One order of summation per
// output element whatever else is in the step.
//   offsets == null: every group has the same `rows` rows (row m is token m), group g reads the columns from
//                    g * a_group on and writes the columns from g * out_group on; blockIdx.z is the group.
//   offsets != null: group g owns the rows offsets[g] .. offsets[g + 1] - 1 (sorted slots); blockIdx.x runs over an upper
//                    bound of all groups' tiles and finds its group by walking the offsets; `src` (optional) maps a
//                    sorted slot to the row of `a` it reads (a token routed to an expert), output rows are the slots.
#define GG_T 64
#define GG_K 16

template <typename T>
__global__ void __launch_bounds__(256)
grouped_gemm_kernel(const T* __restrict__ a, int a_ld, int a_group, const int* __restrict__ src, const T* __restrict__ w,
                    T* __restrict__ out, int out_ld, int out_group, const int* __restrict__ offsets, int groups, int rows,
                    int N, int K, int act) {
    __shared__ float sa[GG_K][GG_T + 4];
    __shared__ float sw[GG_K][GG_T + 4];
    int g, m0, m_end;
    if (offsets == nullptr) {
        g = blockIdx.z; m0 = blockIdx.x * GG_T; m_end = rows;
        if (m0 >= m_end) return;
    } else {
        int tile = blockIdx.x;
        g = 0; m0 = -1; m_end = 0;
        for (int e = 0; e < groups; ++e) {
            const int lo = offsets[e], hi = offsets[e + 1], tiles = (hi - lo + GG_T - 1) / GG_T;
            if (tile < tiles) { g = e; m0 = lo + tile * GG_T; m_end = hi; break; }
            tile -= tiles;
        }
        if (m0 < 0) return;
    }
    const int n0 = blockIdx.y * GG_T;
    const T* wg = w + (size_t)g * N * K;
    const int a_col = offsets == nullptr ? g * a_group : 0, out_col = offsets == nullptr ? g * out_group : 0;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;      // the thread's block: rows ty*4.., columns tx*4..
    // loads: a thread fetches 4 elements of a and 4 of w per step: row lr of the tile, k = lk .. lk+3
    const int lr = threadIdx.x / 4, lk = (threadIdx.x % 4) * 4;
    const int am = m0 + lr;
    const T* arow = nullptr;
    if (am < m_end) arow = a + (size_t)(src ? src[am] : am) * a_ld + a_col;
    const T* wrow = (n0 + lr < N) ? wg + (size_t)(n0 + lr) * K : nullptr;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GG_K) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + lk + u;
            sa[lk + u][lr] = (arow && k < K) ? to_float(arow[k]) : 0.f;
            sw[lk + u][lr] = (wrow && k < K) ? to_float(wrow[k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GG_K; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) { av[u] = sa[k][ty * 4 + u]; wv[u] = sw[k][tx * 4 + u]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
    const int base_act = act & ~ACT_PAIRS;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= m_end) continue;
        T* orow = out + (size_t)m * out_ld + out_col;
        if (act & ACT_PAIRS) {                          // (N is even: a pair lies in one thread's four columns)
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const int n = n0 + tx * 4 + j;
                if (n + 1 < N) orow[n / 2] = from_float<T>(activate(acc[i][j], base_act) * acc[i][j + 1]);
            }
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) orow[n] = from_float<T>(activate(acc[i][j], act));
        }
    }
}

// The same product on the matrix cores (bfloat16, K a multiple of 32, 16-byte aligned rows): both operands have K side by
// side in memory, which is how v_mfma_f32_16x16x32_bf16 wants them, so a lane fetches its 16-byte pieces straight from
// memory (the weights' once per tile of rows, the rows' from the caches) and nothing passes through shared memory.  The
// weights are the first operand, so that a lane ends up with four neighbouring output columns of one row.  A work-group
// of four waves owns a tile of 32 rows x 256 columns (one wave: 32 x 64); few rows per group (a decode step's experts)
// leave half of each product empty, which costs nothing where the weights' stream sets the time.
#define GM_BM 32
#define GM_BN 256

typedef __bf16 gm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gm_f32x4 __attribute__((ext_vector_type(4)));
union GmFrag {
    uint4 u;
    gm_bf16x8 v;
};

__global__ void __launch_bounds__(256)
grouped_gemm_mfma_kernel(const bf16_t* __restrict__ a, int a_ld, int a_group, const int* __restrict__ src, const bf16_t* __restrict__ w,
                         bf16_t* __restrict__ out, int out_ld, int out_group, const int* __restrict__ offsets, int groups, int rows,
                         int N, int K, int act) {
    int g, m0, m_end;
    if (offsets == nullptr) {
        g = blockIdx.z; m0 = blockIdx.x * GM_BM; m_end = rows;
        if (m0 >= m_end) return;
    } else {
        int tile = blockIdx.x;
        g = 0; m0 = -1; m_end = 0;
        for (int e = 0; e < groups; ++e) {
            const int lo = offsets[e], hi = offsets[e + 1], tiles = (hi - lo + GM_BM - 1) / GM_BM;
            if (tile < tiles) { g = e; m0 = lo + tile * GM_BM; m_end = hi; break; }
            tile -= tiles;
        }
        if (m0 < 0) return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.y * GM_BN + wave * 64;
    if (n0 >= N) return;
    const bf16_t* wg = w + (size_t)g * N * K;
    const int a_col = offsets == nullptr ? g * a_group : 0, out_col = offsets == nullptr ? g * out_group : 0;
    // this lane's rows of the two operands: weight row n0 + 16 i + li (clamped), x row of tile row 16 j + li (clamped)
    const bf16_t* wrow[4];
    const bf16_t* xrow[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) wrow[i] = wg + (size_t)min(n0 + 16 * i + li, N - 1) * K + 8 * kg;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int m = min(m0 + 16 * j + li, m_end - 1);
        xrow[j] = a + (size_t)(src ? src[m] : m) * a_ld + a_col + 8 * kg;
    }
    const bool second = m0 + 16 < m_end;                // the tile has rows beyond its first 16
    gm_f32x4 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = gm_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int k = 0; k < K; k += 32) {
        GmFrag wf[4], xf[2];
#pragma unroll
        for (int i = 0; i < 4; ++i) wf[i].u = *(const uint4*)(wrow[i] + k);
        xf[0].u = *(const uint4*)(xrow[0] + k);
        if (second) xf[1].u = *(const uint4*)(xrow[1] + k);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[i][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, xf[0].v, acc[i][0], 0, 0, 0);
            if (second) acc[i][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, xf[1].v, acc[i][1], 0, 0, 0);
        }
    }
    // acc[i][j][v] = out[row 16 j + li][column n0 + 16 i + 4 kg + v]
    const int base_act = act & ~ACT_PAIRS;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int m = m0 + 16 * j + li;
        if (m >= m_end) continue;
        bf16_t* orow = out + (size_t)m * out_ld + out_col;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + 16 * i + 4 * kg;
            if (act & ACT_PAIRS) {                      // a lane's four columns are two pairs: two outputs at column n / 2
#pragma unroll
                for (int v = 0; v < 4; v += 2)
                    if (n + v + 1 < N) orow[(n + v) / 2] = from_float<bf16_t>(activate(acc[i][j][v], base_act) * acc[i][j][v + 1]);
                continue;
            }
            if (n + 3 < N && ((out_ld | out_col) & 3) == 0) {
                union { uint2 u; uint16_t e[4]; } pk;
#pragma unroll
                for (int v = 0; v < 4; ++v) pk.e[v] = from_float<bf16_t>(activate(acc[i][j][v], act)).bits;
                *(uint2*)(orow + n) = pk.u;
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) orow[n + v] = from_float<bf16_t>(activate(acc[i][j][v], act));
            }
        }
    }
}

extern "C" int tl_grouped_gemm(const void* a, int a_ld, int a_group, const void* src, const void* w, void* out, int out_ld, int out_group,
                               const void* offsets, int groups, int rows, int N, int K, int act, int dtype, int general, hipStream_t stream) {
    TL_REQUIRE(groups > 0 && rows >= 0 && N > 0 && K > 0 && a_ld > 0 && out_ld > 0, "grouped_gemm: bad sizes");
    TL_REQUIRE(known_activation(act), "grouped_gemm: unknown activation %d", act);
    TL_REQUIRE(!(act & ACT_PAIRS) || (N % 2 == 0 && out_group == 0), "grouped_gemm: an activation in pairs needs an even number of columns");
    if (rows == 0) return TL_OK;
    // with offsets, `rows` is the number of sorted slots in all groups together: every group may end in a partial tile
    dim3 grid(offsets ? (rows + GG_T - 1) / GG_T + groups : (rows + GG_T - 1) / GG_T, (N + GG_T - 1) / GG_T, offsets ? 1 : groups), block(256);
    const bool aligned = K % 32 == 0 && a_ld % 8 == 0 && a_group % 8 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0 &&
                         ((uintptr_t)out % 8) == 0;
    if (dtype == TL_DT_BF16 && aligned && !general) {
        dim3 mgrid(offsets ? (rows + GM_BM - 1) / GM_BM + groups : (rows + GM_BM - 1) / GM_BM, (N + GM_BN - 1) / GM_BN, offsets ? 1 : groups);
        grouped_gemm_mfma_kernel<<<mgrid, block, 0, stream>>>((const bf16_t*)a, a_ld, a_group, (const int*)src, (const bf16_t*)w, (bf16_t*)out, out_ld,
                                                              out_group, (const int*)offsets, groups, rows, N, K, act);
        TL_CHECK_LAUNCH("grouped_gemm_mfma");
        return TL_OK;
    }
    if (dtype == TL_DT_F32)
        grouped_gemm_kernel<float><<<grid, block, 0, stream>>>((const float*)a, a_ld, a_group, (const int*)src, (const float*)w, (float*)out, out_ld,
                                                               out_group, (const int*)offsets, groups, rows, N, K, act);
    else if (dtype == TL_DT_BF16)
        grouped_gemm_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)a, a_ld, a_group, (const int*)src, (const bf16_t*)w, (bf16_t*)out, out_ld,
                                                                out_group, (const int*)offsets, groups, rows, N, K, act);
    else TL_REQUIRE(false, "grouped_gemm: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("grouped_gemm");
    return TL_OK;
}

// ------------------------------------------------------------------ the router's choice
// Per token (one wave): the `top` best of its `experts` outputs, best first (the lower index wins a tie), and their weights.
//   mode 0: the choice goes by the logits; the weights are the softmax over the chosen logits alone.
//   mode 1: the scores are the softmax over all logits; the choice goes by score + bias[e] (bias optional), the weights are the
//           chosen experts' scores as they are.
//   mode 2: the scores are the logits' sigmoids; the choice goes by score + bias[e] (bias optional), the weights are the chosen
//           experts' scores divided by their sum plus weight_eps.
// In every mode the weights are multiplied by weight_scale at the end.
__global__ void route_topk_kernel(const float* __restrict__ logits, int experts, int top, int mode, const float* __restrict__ bias,
                                  int* __restrict__ chosen, float* __restrict__ weights, int tokens, float weight_scale, float weight_eps) {
    const int t = blockIdx.x * (blockDim.x / TL_WAVE) + threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    if (t >= tokens) return;
    const float* z = logits + (size_t)t * experts;
    float zmax = 0.f, den = 1.f;
    if (mode == 1) {
        float mx = -INFINITY;
        for (int e = lane; e < experts; e += TL_WAVE) mx = fmaxf(mx, z[e]);
        zmax = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < experts; e += TL_WAVE) sum += expf(z[e] - zmax);
        den = wave_sum(sum);
    }
    float first = 0.f, sum = 0.f, mine = 0.f;           // lane j keeps the j-th choice's term
    unsigned long long taken = 0;                       // bit i: this lane's expert lane + 64 * i is chosen already
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY, score = 0.f;
        int at = 0x7fffffff;
        for (int e = lane, i = 0; e < experts; e += TL_WAVE, ++i) {
            float v = z[e], sc = 0.f;
            if (mode == 1) { sc = expf(v - zmax) / den; v = bias ? sc + bias[e] : sc; }
            else if (mode == 2) { sc = 1.f / (1.f + expf(-v)); v = bias ? sc + bias[e] : sc; }
            if (!((taken >> i) & 1ull) && (v > best || (v == best && e < at))) { best = v; at = e; score = sc; }
        }
#pragma unroll
        for (int o = TL_WAVE / 2; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, TL_WAVE);
            const float os = __shfl_xor(score, o, TL_WAVE);
            const int oa = __shfl_xor(at, o, TL_WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; score = os; }
        }
        if (at % TL_WAVE == lane) taken |= 1ull << (at / TL_WAVE);
        if (j == 0) first = best;
        const float p = mode != 0 ? score : expf(best - first);
        sum += p;
        if (lane == j) { chosen[(size_t)t * top + j] = at; mine = p; }
    }
    if (lane < top) weights[(size_t)t * top + lane] = (mode == 1 ? mine : mode == 2 ? mine / (sum + weight_eps) : mine / sum) * weight_scale;
}

// Sort of the (token, choice) pairs by expert, by one work-group: offsets[e] .. offsets[e + 1] - 1 are the slots of
// expert e, slot_token[slot] the token a slot reads, pair_slot[token * top + j] where the pair's output row lies.
__global__ void __launch_bounds__(1024)
route_sort_kernel(const int* __restrict__ chosen, int pairs, int top, int experts, int* __restrict__ offsets,
                  int* __restrict__ slot_token, int* __restrict__ pair_slot) {
    extern __shared__ int cursor[];                     // [experts + 1]
    for (int e = threadIdx.x; e <= experts; e += blockDim.x) cursor[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&cursor[chosen[i] + 1], 1);
    __syncthreads();
    if (threadIdx.x == 0)
        for (int e = 0; e < experts; ++e) cursor[e + 1] += cursor[e];
    __syncthreads();
    for (int e = threadIdx.x; e <= experts; e += blockDim.x) offsets[e] = cursor[e];
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
        const int slot = atomicAdd(&cursor[chosen[i]], 1);
        slot_token[slot] = i / top;
        pair_slot[i] = slot;
    }
}

extern "C" int tl_route(const void* logits, int tokens, int experts, int top, int mode, const void* bias, void* chosen, void* weights,
                        void* offsets, void* slot_token, void* pair_slot, float weight_scale, float weight_eps, hipStream_t stream) {
    TL_REQUIRE(mode >= 0 && mode <= 2, "route: unknown mode %d", mode);
    TL_REQUIRE(tokens >= 0 && experts > 0 && top > 0 && top <= experts && top <= TL_WAVE && experts <= 64 * TL_WAVE, "route: bad sizes (experts %d, top %d)", experts, top);
    TL_REQUIRE((experts + 1) * sizeof(int) <= 64 * 1024, "route: too many experts (%d)", experts);
    if (tokens == 0) return TL_OK;
    route_topk_kernel<<<(tokens + 3) / 4, 4 * TL_WAVE, 0, stream>>>((const float*)logits, experts, top, mode, (const float*)bias, (int*)chosen, (float*)weights, tokens,
                                                                    weight_scale, weight_eps);
    TL_CHECK_LAUNCH("route_topk");
    route_sort_kernel<<<1, 1024, (experts + 1) * sizeof(int), stream>>>((const int*)chosen, tokens * top, top, experts, (int*)offsets,
                                                                       (int*)slot_token, (int*)pair_slot);
    TL_CHECK_LAUNCH("route_sort");
    return TL_OK;
}

// ------------------------------------------------------------------ weighted sum of the chosen experts' outputs
// out[t, :] = sum_j weights[t, j] * y[pair_slot[t * top + j], :], summed in the order of the choices.  With `x`: a pair whose slot is
// offsets[real] or later chose an expert without tensors (an identity expert), and x[t, :] stands in for its row of y.  With `addend`
// (a shared expert's output): out[t, :] += addend[t, :], added last, in float.
template <typename T>
__global__ void combine_kernel(const T* __restrict__ y, const int* __restrict__ pair_slot, const float* __restrict__ weights,
                               T* __restrict__ out, const T* __restrict__ x, const int* __restrict__ offsets, int real, int top, int width,
                               const T* __restrict__ addend) {
    const int t = blockIdx.x;
    const int own_from = x ? offsets[real] : 0x7fffffff;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float a = 0.f;
        for (int j = 0; j < top; ++j) {
            const int slot = pair_slot[(size_t)t * top + j];
            const float v = slot >= own_from ? to_float(x[(size_t)t * width + i]) : to_float(y[(size_t)slot * width + i]);
            a = fmaf(weights[(size_t)t * top + j], v, a);
        }
        if (addend) a += to_float(addend[(size_t)t * width + i]);
        out[(size_t)t * width + i] = from_float<T>(a);
    }
}

extern "C" int tl_combine(const void* y, const void* pair_slot, const void* weights, void* out, const void* x, const void* offsets, int real,
                          int tokens, int top, int width, const void* addend, int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && top > 0 && width > 0 && real >= 0 && (!x || offsets), "combine: bad sizes");
    if (tokens == 0) return TL_OK;
    if (dtype == TL_DT_F32)
        combine_kernel<float><<<tokens, 256, 0, stream>>>((const float*)y, (const int*)pair_slot, (const float*)weights, (float*)out, (const float*)x,
                                                          (const int*)offsets, real, top, width, (const float*)addend);
    else if (dtype == TL_DT_BF16)
        combine_kernel<bf16_t><<<tokens, 256, 0, stream>>>((const bf16_t*)y, (const int*)pair_slot, (const float*)weights, (bf16_t*)out, (const bf16_t*)x,
                                                           (const int*)offsets, real, top, width, (const bf16_t*)addend);
    else TL_REQUIRE(false, "combine: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("combine");
    return TL_OK;
}

// ------------------------------------------------------------------ elementwise activation, in place
template <typename T>
__global__ void activation_kernel(T* __restrict__ x, size_t n, int act) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        x[i] = from_float<T>(activate(to_float(x[i]), act));
}

extern "C" int tl_activation(void* x, long n, int act, int dtype, hipStream_t stream) {
    TL_REQUIRE(n >= 0 && known_activation(act) && !(act & ACT_PAIRS), "activation: bad arguments");
    if (n == 0 || act == ACT_NONE) return TL_OK;
    const int blocks = (int)((n + 1023) / 1024 < 8192 ? (n + 1023) / 1024 : 8192);
    if (dtype == TL_DT_F32) activation_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, (size_t)n, act);
    else if (dtype == TL_DT_BF16) activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, (size_t)n, act);
    else TL_REQUIRE(false, "activation: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("activation");
    return TL_OK;
}
