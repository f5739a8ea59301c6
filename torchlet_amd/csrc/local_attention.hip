// Attention over a paged cache whose keys and values differ in size (dim and vdim numbers per head), with soft-capped scores and a
// local mask: a query at position p reads the keys j <= p of its own chunk (j / chunk == p / chunk, chunks counted from position 0)
// and, with a window, j > p - window.  Scores, softmax and the weighted sum are float whatever the activation type.
//   k_plane [pages, kv_heads, page_size, dim], v_plane [pages, kv_heads, vdim, page_size] (the values of a page lie transposed, so
//   that eight neighbouring keys' values of one column are 16 bytes side by side, which is how the matrix cores want them); key j
//   of a request lies in slot j % page_size of page block_table[request][j / page_size].
// Two more mechanisms, each switched on by its operand.  A sink: the softmax's denominator also holds exp(sink[head]), which has neither
// key nor value and is not scaled.  Pooled blocks: beside a window of `window` tokens a query at position p reads one key and one
// value for every block of `pool` positions that lies wholly before its window, blocks 0 .. (p - window + 1) / pool - 1; block b's key
// and value are the means of the cached keys and values of the positions b * pool .. b * pool + pool - 1 and lie, as a token's would, in
// row b of planes of their own with a block table of their own (pool_blocks_kernel makes them when a step brings a block's last token).
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
        v_plane[(((size_t)page * kv_heads + g) * vdim + d) * page_size + slot] = v[(size_t)t * v_ld + i];
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
    int keep_first;          // beside a window: the positions 0 .. keep_first - 1 are read by every later query, at their own places
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
                       LocalMask mask, float gain, const float* __restrict__ sink, const T* __restrict__ pk_plane, const T* __restrict__ pv_plane,
                       const int* __restrict__ pool_table, int pool_table_ld, int pool) {
    __shared__ float sq[LA_MAX_DIM];
    __shared__ float sm[LA_WAVES], sl[LA_WAVES];
    __shared__ float sacc[LA_WAVES][LA_MAX_DIM];
    const int t = blockIdx.x, head = blockIdx.y;
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    const int g = head / (heads / kv_heads);
    const int p = positions[t];
    const int lo = mask.first(p);
    const int* table = block_table + (size_t)token_req[t] * table_ld;
    const int* ptable = pool > 0 ? pool_table + (size_t)token_req[t] * pool_table_ld : nullptr;
    const int npool = (pool > 0 && mask.window > 0) ? max(0, p - mask.window + 1) / pool : 0;      // pooled blocks: keys 0 .. npool - 1 of this query
    for (int d = threadIdx.x; d < dim; d += blockDim.x) sq[d] = to_float(q[(size_t)t * q_ld + head * dim + d]) * scale;
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[LA_COLS];
#pragma unroll
    for (int c = 0; c < LA_COLS; ++c) acc[c] = 0.f;
    const int nkept = min(mask.keep_first, lo);          // kept first tokens that lie before the window: keys npool .. npool + nkept - 1
    const int nkeys = npool + nkept + p - lo + 1;
    for (int b = wave; b * TL_WAVE < nkeys; b += LA_WAVES) {
        const int u = b * TL_WAVE + lane;                // pooled blocks first, then the kept first tokens, then the tokens lo .. p
        const bool ok = u < nkeys;
        float s = -INFINITY;
        const T* vr0 = v_plane;                          // the key's values: column c at vr0[c * page_size]
        if (ok) {
            const bool pooled = u < npool;
            const int j = pooled ? u : (u < npool + nkept ? u - npool : lo + u - npool - nkept);
            const int page = (pooled ? ptable : table)[j / page_size];
            const size_t at = (size_t)page * kv_heads + g;
            const int slot = j % page_size;
            const T* kr = (pooled ? pk_plane : k_plane) + (at * page_size + slot) * dim;
            vr0 = (pooled ? pv_plane : v_plane) + at * vdim * page_size + slot;
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
        const int nb = min(TL_WAVE, nkeys - b * TL_WAVE);
        const unsigned long long vaddr = (unsigned long long)(uintptr_t)vr0;
        for (int i = 0; i < nb; ++i) {
            const float wi = __shfl(w, i, TL_WAVE);
            const unsigned long long ai = ((unsigned long long)(unsigned)__shfl((int)(vaddr >> 32), i, TL_WAVE) << 32) | (unsigned)__shfl((int)vaddr, i, TL_WAVE);
            const T* vr = (const T*)(uintptr_t)ai;
#pragma unroll
            for (int c = 0; c < LA_COLS; ++c) {
                const int col = lane + c * TL_WAVE;
                if (col < vdim) acc[c] = fmaf(wi, to_float(vr[(size_t)col * page_size]), acc[c]);
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
        if (sink) top = fmaxf(top, sink[head]);
        float den = 0.f, f[LA_WAVES];
        for (int w = 0; w < LA_WAVES; ++w) {
            f[w] = sl[w] > 0.f ? expf(sm[w] - top) : 0.f;       // a wave without keys: no share
            den = fmaf(sl[w], f[w], den);
        }
        if (sink) den += expf(sink[head] - top);
        const float norm = gain / den;
        for (int col = lane; col < vdim; col += TL_WAVE) {
            float o = 0.f;
            for (int w = 0; w < LA_WAVES; ++w) o = fmaf(sacc[w][col], f[w], o);
            out[(size_t)t * out_ld + head * vdim + col] = from_float<T>(o * norm);
        }
    }
}


// ------------------------------------------------------------------ the matrix-core kernel (bfloat16, prompts)
// One work-group of four waves per tile of 16 consecutive tokens of a request and query head.  The tile's keys come in steps of 32, dealt
// to the waves in turn (step i to wave i % 4: a matter of the positions alone), so that the longest tile of a step, whose time is the
// chain of its steps, takes a quarter of them per wave; the four waves' running maxima, sums and outputs are joined through shared
// memory at the end.  The operands do not pass through shared memory: with v_mfma_f32_16x16x32_bf16 the first
// operand's lane holds 8 neighbouring k of one row, which for keys (rows of K, k along dim), queries (rows of Q, k along dim) and
// transposed values (rows of V^T, k along the keys of a page) are 16 bytes side by side in memory.
//   scores, transposed: S^T[key][token] = K Q^T.  A lane ends up with one token (lane % 16) and four keys (rows 4 q .. 4 q + 3, q = lane / 16)
//   per product.  A step takes 32 keys in two products whose rows are keys base + 8 (r / 4) + r % 4 and that plus 4, so a lane holds
//   the keys base + 8 q .. 8 q + 7 of its token: exactly the 8 neighbouring k of the second operand of
//   O^T[column][token] += V^T[column][key] P^T[key][token], with no exchange between lanes.
// Cap, mask, running maximum and sum are per token, that is per lane, with the maximum and the final sum joined across the four
// lanes of a token.  Weights are rounded to bfloat16 for the second product; sums are float.
typedef __bf16 la_bf16x8 __attribute__((ext_vector_type(8)));
typedef float la_f32x4 __attribute__((ext_vector_type(4)));
union LaFrag {
    uint4 u;
    la_bf16x8 v;
    uint16_t e[8];
};
#define LAM_TOKENS 16
#define LAM_KEYS 32
#define LAM_WAVES 4
#define LAM_STRIDE (LAM_WAVES * LAM_KEYS)      // keys from one step of a wave to its next

// The hardware's own 2^x and 1 / x (about one unit in the last place each): a tile's time is these, eight scores to a lane and step.
#define LA_LOG2E 1.4426950408889634f

__device__ __forceinline__ float cap_score_fast(float s, float cap, float two_log2e_over_cap) {
    if (cap <= 0.f) return s;
    // cap * tanh(s / cap) with tanh(x) = 1 - 2 / (e^(2 x) + 1); beyond |x| = 15 it is +-1 to the last bit
    const float e = __builtin_amdgcn_exp2f(fminf(fmaxf(s * two_log2e_over_cap, -43.f), 43.f));
    return cap * (1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f));
}

template <int DK, int DV>          // dim / 32 and vdim / 16
__global__ void __launch_bounds__(256)
local_attention_mfma_kernel(const bf16_t* __restrict__ q, int q_ld, bf16_t* __restrict__ out, int out_ld, const bf16_t* __restrict__ k_plane,
                            const bf16_t* __restrict__ v_plane, const int* __restrict__ block_table, int table_ld, int table_width,
                            const int* __restrict__ req_indptr, const int* __restrict__ ctx_lens, const int* __restrict__ tile_req,
                            const int* __restrict__ tile_tok0, int heads, int kv_heads, int page_size, float scale, float cap,
                            LocalMask mask, float gain, const float* __restrict__ sink, const bf16_t* __restrict__ pk_plane,
                            const bf16_t* __restrict__ pv_plane, const int* __restrict__ pool_table, int pool_table_ld, int pool_table_width, int pool) {
    constexpr int dim = DK * 32, vdim = DV * 16;
    extern __shared__ float la_smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, kq = lane >> 4;
    const int head = blockIdx.y;
    const int tile = blockIdx.x;
    const int req = tile_req ? tile_req[tile] : tile;
    const int first = req_indptr[req], n_new = req_indptr[req + 1] - first;
    const int tok0 = tile_tok0 ? tile_tok0[tile] : 0;
    const int n_tile = min(LAM_TOKENS, n_new - tok0);            // tokens of this tile
    if (n_tile <= 0) return;
    const int g = head / (heads / kv_heads);
    const int p0 = ctx_lens[req] + tok0;                         // position of the tile's first token
    const int my_tok = min(li, n_tile - 1);                      // (lanes beyond the tile's tokens repeat its last one and store nothing)
    const int my_p = p0 + my_tok, my_lo = mask.first(my_p);
    const int* table = block_table + (size_t)req * table_ld;
    const float inv_cap = cap > 0.f ? 2.f * LA_LOG2E / cap : 0.f;
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    const int page_shift = __ffs(page_size) - 1;
    auto page_of = [&](int key) { return pow2 ? key >> page_shift : key / page_size; };
    auto slot_of = [&](int key) { return pow2 ? key & (page_size - 1) : key % page_size; };

    LaFrag qf[DK];
    {
        const bf16_t* qrow = q + (size_t)(first + tok0 + my_tok) * q_ld + head * dim + 8 * kq;
#pragma unroll
        for (int s = 0; s < DK; ++s) qf[s].u = *(const uint4*)(qrow + 32 * s);
    }
    la_f32x4 acc[DV];
#pragma unroll
    for (int j = 0; j < DV; ++j) acc[j] = la_f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    const int p_last = p0 + n_tile - 1;
    // rows of the two score products that this lane fetches: keys base + 8 (li / 4) + li % 4 (+ 4)
    const int krow = 8 * (li >> 2) + (li & 3);
    // One pass over a stretch of keys lo_valid .. hi_valid of planes kp / vp (the tokens of the tile's reach, or the pooled blocks before its
    // window), of which this lane's token reads my_first .. my_last.  The running maximum, sum and output carry over from pass to pass.
    auto run = [&](const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp, const int* __restrict__ tbl, int tbl_width, int lo_valid, int hi_valid,
                   int my_first, int my_last) {
        const int base0 = lo_valid / LAM_KEYS * LAM_KEYS;
        if (base0 + LAM_KEYS * wave > hi_valid) return;
        // The pages of up to 64 blocks of the request lie in a register across the wave (lane i: block tab_first + i) and are read from
        // there, so that no fetch waits for a look-up in memory; the window moves on every 64 blocks.
        int tab_first = page_of(base0);
        int tab_reg = tbl[min(tab_first + lane, tbl_width - 1)];
        auto page_at = [&](int key) { return __shfl(tab_reg, page_of(key) - tab_first, TL_WAVE); };
        // The keys and values of a step are fetched one step ahead, while the step before is worked on.
        LaFrag a0[DK], a1[DK], va[DV], vb[DV];
        auto fetch = [&](int base, LaFrag (&vf)[DV]) {
            if (page_of(base + LAM_KEYS - 1) - tab_first >= TL_WAVE) {            // (the same for every lane)
                tab_first = page_of(base);
                tab_reg = tbl[min(tab_first + lane, tbl_width - 1)];
            }
            // keys: rows base + krow and base + krow + 4 (clamped into what exists: masked below)
            const int key0 = max(min(base + krow, hi_valid), lo_valid), key1 = max(min(base + krow + 4, hi_valid), lo_valid);
            const bf16_t* k0 = kp + (((size_t)page_at(key0) * kv_heads + g) * page_size + slot_of(key0)) * dim + 8 * kq;
            const bf16_t* k1 = kp + (((size_t)page_at(key1) * kv_heads + g) * page_size + slot_of(key1)) * dim + 8 * kq;
#pragma unroll
            for (int s = 0; s < DK; ++s) { a0[s].u = *(const uint4*)(k0 + 32 * s); a1[s].u = *(const uint4*)(k1 + 32 * s); }
            // values, transposed: row = column of the values, k = keys base + 8 kq .. + 7 (one page: page_size % 8 == 0)
            const int key = base + 8 * kq;
            const int kc = max(min(key, hi_valid), lo_valid);
            const bf16_t* vt = vp + (((size_t)page_at(kc) * kv_heads + g) * vdim + li) * page_size + slot_of(key);
#pragma unroll
            for (int j = 0; j < DV; ++j) vf[j].u = *(const uint4*)(vt + (size_t)16 * j * page_size);      // (never conditional: nothing waits for it here)
        };
        auto step = [&](int base, LaFrag (&vf)[DV], LaFrag (&vnext)[DV]) {
            // ---- scores of 32 keys
            la_f32x4 s0 = la_f32x4{0.f, 0.f, 0.f, 0.f}, s1 = la_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < DK; ++s) {
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[s].v, qf[s].v, s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[s].v, qf[s].v, s1, 0, 0, 0);
            }
            if (base + LAM_STRIDE <= hi_valid) fetch(base + LAM_STRIDE, vnext);
            // ---- cap, mask, running maximum (scores in units of log 2 from here on, so that the weights are plain powers of two)
            float sc[8];
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = base + 8 * kq + e;
                const float raw = (e < 4 ? s0[e] : s1[e - 4]) * scale;
                sc[e] = (key <= my_last && key >= my_first) ? cap_score_fast(raw, cap, inv_cap) * LA_LOG2E : -INFINITY;
                mx = fmaxf(mx, sc[e]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TL_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TL_WAVE));
            const float m_new = fmaxf(m, mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;   // a token that has seen no key yet
            const float keep = __builtin_amdgcn_exp2f(m - m_use);   // (0 while m is -inf)
            m = m_new;
            LaFrag pf;
            float psum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = __builtin_amdgcn_exp2f(sc[e] - m_use);
                const bf16_t wb = from_float<bf16_t>(w);
                pf.e[e] = wb.bits;
                psum += to_float(wb);                               // the sum of what the second product sees
            }
            l = l * keep + psum;
            // places no token has written yet, or whose page is gone, may hold anything: their values count as zero (first and last steps only)
            const int vkey = base + 8 * kq;
            if (vkey + 7 > hi_valid || vkey < lo_valid) {
#pragma unroll
                for (int j = 0; j < DV; ++j)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (vkey + e > hi_valid || vkey + e < lo_valid) vf[j].e[e] = 0;
            }
            if (__any(keep != 1.f)) {                               // (the maxima settle after a tile's first steps)
#pragma unroll
                for (int j = 0; j < DV; ++j) { acc[j][0] *= keep; acc[j][1] *= keep; acc[j][2] *= keep; acc[j][3] *= keep; }
            }
#pragma unroll
            for (int j = 0; j < DV; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j].v, pf.v, acc[j], 0, 0, 0);
        };
        fetch(base0 + LAM_KEYS * wave, va);
        for (int base = base0 + LAM_KEYS * wave; base <= hi_valid; base += 2 * LAM_STRIDE) {
            step(base, va, vb);
            if (base + LAM_STRIDE <= hi_valid) step(base + LAM_STRIDE, vb, va);
        }
    };
    if (pool > 0 && mask.window > 0) {
        // the pooled blocks that lie wholly before a token's window: 0 .. (p - window + 1) / pool - 1; the tile's last token reads the most
        const int n_tile_blocks = max(0, p_last - mask.window + 1) / pool, n_my_blocks = max(0, my_p - mask.window + 1) / pool;
        if (n_tile_blocks > 0)
            run(pk_plane, pv_plane, pool_table + (size_t)req * pool_table_ld, pool_table_width, 0, n_tile_blocks - 1, 0, n_my_blocks - 1);
    }
    if (mask.keep_first > 0 && mask.window > 0) {
        // the kept first tokens that lie before a token's window: 0 .. min(keep_first, its window's start) - 1; the tile's last token reads the most
        const int n_tile_kept = min(mask.keep_first, mask.first(p_last)), n_my_kept = min(mask.keep_first, my_lo);
        if (n_tile_kept > 0) run(k_plane, v_plane, table, table_width, 0, n_tile_kept - 1, 0, n_my_kept - 1);
    }
    // the first token reads furthest back; pages before may be gone
    run(k_plane, v_plane, table, table_width, mask.first(p0), p_last, my_lo, my_p);
    l += __shfl_xor(l, 16, TL_WAVE);
    l += __shfl_xor(l, 32, TL_WAVE);
    // ---- the four waves' shares are joined: per token the maxima, the sums and the outputs, in the order of the waves
    float* sm_m = la_smem;                              // [4][16], in units of log 2
    float* sm_l = sm_m + LAM_WAVES * LAM_TOKENS;        // [4][16]
    float* sm_o = sm_l + LAM_WAVES * LAM_TOKENS;        // [4][16][vdim]
    if (kq == 0) { sm_m[wave * LAM_TOKENS + li] = m; sm_l[wave * LAM_TOKENS + li] = l; }
    // acc[j][v] = O[token li][column 16 j + 4 kq + v]
#pragma unroll
    for (int j = 0; j < DV; ++j)
        *(float4*)(sm_o + ((size_t)wave * LAM_TOKENS + li) * vdim + 16 * j + 4 * kq) = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
    __syncthreads();
    for (int idx = threadIdx.x; idx < n_tile * vdim; idx += blockDim.x) {
        const int tok = idx / vdim, col = idx % vdim;
        float top = sm_m[tok];
#pragma unroll
        for (int w = 1; w < LAM_WAVES; ++w) top = fmaxf(top, sm_m[w * LAM_TOKENS + tok]);
        const float sink2 = sink ? sink[head] * LA_LOG2E : -INFINITY;       // in units of log 2, like the maxima
        top = fmaxf(top, sink2);
        float den = __builtin_amdgcn_exp2f(sink2 - top), o = 0.f;           // (0 without a sink)
#pragma unroll
        for (int w = 0; w < LAM_WAVES; ++w) {
            const float f = __builtin_amdgcn_exp2f(sm_m[w * LAM_TOKENS + tok] - top);        // (0 for a wave that saw no key of this token)
            den = fmaf(sm_l[w * LAM_TOKENS + tok], f, den);
            o = fmaf(sm_o[((size_t)w * LAM_TOKENS + tok) * vdim + col], f, o);
        }
        out[(size_t)(first + tok0 + tok) * out_ld + head * vdim + col] = from_float<bf16_t>(o * (gain / den));
    }
}

template <int DK, int DV>
static void launch_local_mfma(const void* q, int q_ld, void* out, int out_ld, const void* k_plane, const void* v_plane, const void* block_table,
                              int table_ld, int table_width, const void* req_indptr, const void* ctx_lens, const void* tile_req,
                              const void* tile_tok0, int tiles, int heads, int kv_heads, int page_size, float scale, float cap, LocalMask mask,
                              float gain, const void* sink, const void* pk_plane, const void* pv_plane, const void* pool_table, int pool_table_ld,
                              int pool_table_width, int pool, hipStream_t stream) {
    dim3 grid(tiles, heads), block(LAM_WAVES * TL_WAVE);
    const size_t smem = sizeof(float) * LAM_WAVES * LAM_TOKENS * (2 + DV * 16);
    auto kernel = local_attention_mfma_kernel<DK, DV>;
    static bool raised = false;                      // (per instance of the template)
    if (smem > 48 * 1024 && !raised) {
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        raised = true;
    }
    kernel<<<grid, block, smem, stream>>>((const bf16_t*)q, q_ld, (bf16_t*)out, out_ld, (const bf16_t*)k_plane, (const bf16_t*)v_plane,
        (const int*)block_table, table_ld, table_width, (const int*)req_indptr, (const int*)ctx_lens, (const int*)tile_req, (const int*)tile_tok0,
        heads, kv_heads, page_size, scale, cap, mask, gain, (const float*)sink, (const bf16_t*)pk_plane, (const bf16_t*)pv_plane, (const int*)pool_table,
        pool_table_ld, pool_table_width, pool);
}

// Whether the matrix-core kernel is built for these sizes.
extern "C" int tl_local_attention_mfma_fits(int dim, int vdim, int page_size) {
    const bool dk = dim == 32 || dim == 64 || dim == 96 || dim == 128 || dim == 192 || dim == 256;
    const bool dv = vdim == 16 || vdim == 32 || vdim == 64 || vdim == 96 || vdim == 128 || vdim == 192 || vdim == 256;
    return dk && dv && page_size % 8 == 0;
}

// Tiles of up to 16 consecutive tokens of one request: tile i belongs to request tile_req[i] (null: request i) and starts at that
// request's token tile_tok0[i] of the step (null: 0).
extern "C" int tl_local_attention_tiles(const void* q, int q_ld, void* out, int out_ld, const void* k_plane, const void* v_plane, int pages,
                                        const void* block_table, int table_ld, int table_width, const void* req_indptr, const void* ctx_lens,
                                        const void* tile_req, const void* tile_tok0, int tiles, int heads, int kv_heads, int dim, int vdim,
                                        int page_size, float scale, float cap, int chunk, int window, float gain, const void* sink,
                                        const void* pk_plane, const void* pv_plane, const void* pool_table, int pool_table_ld, int pool_table_width,
                                        int pool, int keep_first, hipStream_t stream) {
    TL_REQUIRE(keep_first >= 0 && (keep_first == 0 || (window > 0 && chunk == 0)), "local_attention_tiles: kept first tokens stand beside a window, without chunks");
    TL_REQUIRE(pool >= 0 && (pool == 0 || (window > 0 && pk_plane && pv_plane && pool_table && pool_table_ld >= pool_table_width && pool_table_width > 0)),
               "local_attention_tiles: pooled blocks need a window, their planes and their block table");
    TL_REQUIRE(tiles >= 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && page_size > 0, "local_attention_tiles: bad sizes");
    TL_REQUIRE(tl_local_attention_mfma_fits(dim, vdim, page_size), "local_attention_tiles: not built for heads of %d / %d numbers in pages of %d", dim, vdim, page_size);
    TL_REQUIRE(q_ld >= heads * dim && q_ld % 8 == 0 && ((uintptr_t)q & 15) == 0 && out_ld >= heads * vdim && table_ld >= table_width && chunk >= 0 && window >= 0,
               "local_attention_tiles: rows too short or not aligned");
    if (tiles == 0) return TL_OK;
    const LocalMask mask{chunk, window, keep_first};
#define TL_LAM(DK, DV)                                                                                                                      \
    launch_local_mfma<DK, DV>(q, q_ld, out, out_ld, k_plane, v_plane, block_table, table_ld, table_width, req_indptr, ctx_lens, tile_req,  \
                              tile_tok0, tiles, heads, kv_heads, page_size, scale, cap, mask, gain, sink, pk_plane, pv_plane, pool_table,        \
                              pool_table_ld, pool_table_width, pool, stream)
#define TL_LAM_V(DK)                                     \
    switch (vdim) {                                      \
        case 16: TL_LAM(DK, 1); break;                   \
        case 32: TL_LAM(DK, 2); break;                   \
        case 64: TL_LAM(DK, 4); break;                   \
        case 96: TL_LAM(DK, 6); break;                   \
        case 128: TL_LAM(DK, 8); break;                  \
        case 192: TL_LAM(DK, 12); break;                 \
        default: TL_LAM(DK, 16); break;                  \
    }
    switch (dim) {
        case 32: TL_LAM_V(1) break;
        case 64: TL_LAM_V(2) break;
        case 96: TL_LAM_V(3) break;
        case 128: TL_LAM_V(4) break;
        case 192: TL_LAM_V(6) break;
        default: TL_LAM_V(8) break;
    }
#undef TL_LAM_V
#undef TL_LAM
    TL_CHECK_LAUNCH("local_attention_mfma");
    return TL_OK;
}

extern "C" int tl_local_attention(const void* q, int q_ld, void* out, int out_ld, const void* k_plane, const void* v_plane, int pages,
                                  const void* block_table, int table_ld, int table_width, const void* token_req, const void* positions,
                                  int tokens, int heads, int kv_heads, int dim, int vdim, int page_size, float scale, float cap, int chunk,
                                  int window, float gain, const void* sink, const void* pk_plane, const void* pv_plane, const void* pool_table,
                                  int pool_table_ld, int pool, int keep_first, int dtype, hipStream_t stream) {
    TL_REQUIRE(keep_first >= 0 && (keep_first == 0 || (window > 0 && chunk == 0)), "local_attention: kept first tokens stand beside a window, without chunks");
    TL_REQUIRE(pool >= 0 && (pool == 0 || (window > 0 && pk_plane && pv_plane && pool_table)), "local_attention: pooled blocks need a window, their planes and their block table");
    TL_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && page_size > 0, "local_attention: bad sizes");
    TL_REQUIRE(dim <= LA_MAX_DIM && vdim <= LA_MAX_DIM, "local_attention: built for heads of up to %d numbers, got %d / %d", LA_MAX_DIM, dim, vdim);
    TL_REQUIRE(q_ld >= heads * dim && out_ld >= heads * vdim && table_ld >= table_width && chunk >= 0 && window >= 0, "local_attention: rows too short");
    TL_REQUIRE(heads <= 65535, "local_attention: too many heads");
    if (tokens == 0) return TL_OK;
    const LocalMask mask{chunk, window, keep_first};
    dim3 grid(tokens, heads), block(LA_WAVES * TL_WAVE);
    if (dtype == TL_DT_F32)
        local_attention_kernel<float><<<grid, block, 0, stream>>>((const float*)q, q_ld, (float*)out, out_ld, (const float*)k_plane, (const float*)v_plane,
            (const int*)block_table, table_ld, (const int*)token_req, (const int*)positions, heads, kv_heads, dim, vdim, page_size, scale, cap, mask, gain,
            (const float*)sink, (const float*)pk_plane, (const float*)pv_plane, (const int*)pool_table, pool_table_ld, pool);
    else if (dtype == TL_DT_BF16)
        local_attention_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)q, q_ld, (bf16_t*)out, out_ld, (const bf16_t*)k_plane, (const bf16_t*)v_plane,
            (const int*)block_table, table_ld, (const int*)token_req, (const int*)positions, heads, kv_heads, dim, vdim, page_size, scale, cap, mask, gain,
            (const float*)sink, (const bf16_t*)pk_plane, (const bf16_t*)pv_plane, (const int*)pool_table, pool_table_ld, pool);
    else TL_REQUIRE(false, "local_attention: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("local_attention");
    return TL_OK;
}

// ------------------------------------------------------------------ pooled blocks
// Block b of a request (positions b * pool .. b * pool + pool - 1) gets its pooled key and value, the means of its cached keys and values,
// in the step that brings its last token: the blocks ctx / pool .. (ctx + n) / pool - 1 of a request that held ctx tokens and gets n.  One
// wave per such block, key/value head and 64 columns of keys-and-values side by side (a lane owns a column and walks the block's
// positions); sums in float in the order of the positions, one rounding.  Pooled rows lie in planes laid out like the tokens' (values
// transposed) under a block table of their own, block b in row b; what would go to page 0 is dropped.
template <typename T>
__global__ void __launch_bounds__(TL_WAVE)
pool_blocks_kernel(const T* __restrict__ k_plane, const T* __restrict__ v_plane, const int* __restrict__ block_table, int table_ld,
                   int table_width, T* __restrict__ pk_plane, T* __restrict__ pv_plane, const int* __restrict__ pool_table,
                   int pool_table_ld, int pool_table_width, const int* __restrict__ req_indptr, const int* __restrict__ ctx_lens,
                   int kv_heads, int dim, int vdim, int pages, int pool_pages, int page_size, int pool) {
    const int r = blockIdx.y;
    const int ctx = ctx_lens[r], n = req_indptr[r + 1] - req_indptr[r];
    const int b = ctx / pool + blockIdx.x;
    if (n <= 0 || b >= (ctx + n) / pool) return;
    const int pb = b / page_size;
    if (pb >= pool_table_width) return;
    const int ppage = pool_table[(size_t)r * pool_table_ld + pb];
    if (ppage <= 0 || ppage >= pool_pages) return;
    const int pslot = b % page_size;
    const int* table = block_table + (size_t)r * table_ld;
    const int chunks = (dim + vdim + TL_WAVE - 1) / TL_WAVE;
    const int g = blockIdx.z / chunks, e = (blockIdx.z % chunks) * TL_WAVE + threadIdx.x;
    if (e >= dim + vdim) return;
    const bool is_key = e < dim;
    const int d = is_key ? e : e - dim;
    float sum = 0.f;
    for (int j = 0; j < pool; ++j) {
        const int key = b * pool + j, blk = key / page_size, slot = key % page_size;
        const int page = blk < table_width ? table[blk] : 0;
        if (page <= 0 || page >= pages) continue;          // (a block's tokens are all held when its last one arrives)
        sum += is_key ? to_float(k_plane[(((size_t)page * kv_heads + g) * page_size + slot) * dim + d])
                      : to_float(v_plane[(((size_t)page * kv_heads + g) * vdim + d) * page_size + slot]);
    }
    const float mean = sum / (float)pool;
    if (is_key) pk_plane[(((size_t)ppage * kv_heads + g) * page_size + pslot) * dim + d] = from_float<T>(mean);
    else pv_plane[(((size_t)ppage * kv_heads + g) * vdim + d) * page_size + pslot] = from_float<T>(mean);
}

// `most_blocks`: an upper bound of the blocks one request completes in the step (its longest portion / pool + 1).
extern "C" int tl_pool_blocks(const void* k_plane, const void* v_plane, int pages, const void* block_table, int table_ld, int table_width,
                              void* pk_plane, void* pv_plane, int pool_pages, const void* pool_table, int pool_table_ld, int pool_table_width,
                              const void* req_indptr, const void* ctx_lens, int requests, int most_blocks, int kv_heads, int dim, int vdim,
                              int page_size, int pool, int dtype, hipStream_t stream) {
    TL_REQUIRE(requests >= 0 && requests <= 65535 && most_blocks >= 0 && kv_heads > 0 && dim > 0 && vdim > 0 && page_size > 0 && pool > 0 && pages > 0 && pool_pages > 0,
               "pool_blocks: bad sizes");
    TL_REQUIRE(table_ld >= table_width && pool_table_ld >= pool_table_width && table_width > 0 && pool_table_width > 0, "pool_blocks: block tables too short");
    if (requests == 0 || most_blocks == 0) return TL_OK;
    const int chunks = (dim + vdim + TL_WAVE - 1) / TL_WAVE;
    TL_REQUIRE((long)kv_heads * chunks <= 65535, "pool_blocks: too many heads");
    dim3 grid(most_blocks, requests, kv_heads * chunks), block(TL_WAVE);
    if (dtype == TL_DT_F32)
        pool_blocks_kernel<float><<<grid, block, 0, stream>>>((const float*)k_plane, (const float*)v_plane, (const int*)block_table, table_ld, table_width,
            (float*)pk_plane, (float*)pv_plane, (const int*)pool_table, pool_table_ld, pool_table_width, (const int*)req_indptr, (const int*)ctx_lens,
            kv_heads, dim, vdim, pages, pool_pages, page_size, pool);
    else if (dtype == TL_DT_BF16)
        pool_blocks_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)k_plane, (const bf16_t*)v_plane, (const int*)block_table, table_ld, table_width,
            (bf16_t*)pk_plane, (bf16_t*)pv_plane, (const int*)pool_table, pool_table_ld, pool_table_width, (const int*)req_indptr, (const int*)ctx_lens,
            kv_heads, dim, vdim, pages, pool_pages, page_size, pool);
    else TL_REQUIRE(false, "pool_blocks: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("pool_blocks");
    return TL_OK;
}

// ------------------------------------------------------------------ norm per head and rotation, in place
// x [T, ld] holds per token heads_a + heads_b heads of `dim` numbers side by side (queries, then keys).  One wave per token and head, in float:
//   norm (norm_a / norm_b != null): v <- v / sqrt(mean(v^2) + eps) * w[d], w = norm_a for the first heads_a heads, norm_b for the others;
//   rotation (inv_freq != null) of the first `dims` numbers by angle_i = float(position) * inv_freq[i]: pair (2i, 2i + 1), or, `halves`,
//   pair (i, i + dims / 2); (u, v) <- (u cos - v sin, v cos + u sin).  What lies beyond `dims` is not turned.  One rounding at the end.
// `raw_b` (optional, [T, raw_ld]): the heads_b heads as they come, before norm and rotation, are copied there (values that are the keys
// as projected).
#define HNR_WAVES 4
template <typename T>
__global__ void __launch_bounds__(HNR_WAVES * TL_WAVE)
head_norm_rotate_kernel(T* __restrict__ x, int ld, int tokens, int heads_a, int heads_b, int dim, const float* __restrict__ norm_a,
                        const float* __restrict__ norm_b, float eps, const int* __restrict__ positions, const float* __restrict__ inv_freq,
                        int dims, int halves, T* __restrict__ raw_b, int raw_ld) {
    __shared__ float sv[HNR_WAVES][LA_MAX_DIM];
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    const int heads = heads_a + heads_b;
    const long item = (long)blockIdx.x * HNR_WAVES + wave;
    const bool live = item < (long)tokens * heads;
    const int t = live ? (int)(item / heads) : 0, h = live ? (int)(item % heads) : 0;
    T* row = x + (size_t)t * ld + (size_t)h * dim;
    float* v = sv[wave];
    const float* w = h < heads_a ? norm_a : norm_b;
    float ss = 0.f;
    if (live) {
        T* raw = (raw_b && h >= heads_a) ? raw_b + (size_t)t * raw_ld + (size_t)(h - heads_a) * dim : nullptr;
        for (int d = lane; d < dim; d += TL_WAVE) {
            const T x0 = row[d];
            if (raw) raw[d] = x0;
            const float a = to_float(x0); v[d] = a; ss = fmaf(a, a, ss);
        }
    }
    ss = wave_sum(ss);
    __syncthreads();
    if (live && w) {
        const float inv = 1.f / sqrtf(ss / (float)dim + eps);
        for (int d = lane; d < dim; d += TL_WAVE) v[d] = v[d] * inv * w[d];
    }
    __syncthreads();
    if (live && inv_freq) {
        const float pos = (float)positions[t];
        for (int i = lane; i < dims / 2; i += TL_WAVE) {
            const int ia = halves ? i : 2 * i, ib = halves ? i + dims / 2 : 2 * i + 1;
            float sn, c;
            sincosf(pos * inv_freq[i], &sn, &c);
            const float a = v[ia], b = v[ib];
            v[ia] = __fmaf_rn(a, c, -__fmul_rn(b, sn));
            v[ib] = __fmaf_rn(b, c, __fmul_rn(a, sn));
        }
    }
    __syncthreads();
    if (live)
        for (int d = lane; d < dim; d += TL_WAVE) row[d] = from_float<T>(v[d]);
}

extern "C" int tl_head_norm_rotate(void* x, int ld, int tokens, int heads_a, int heads_b, int dim, const void* norm_a, const void* norm_b, float eps,
                                   const void* positions, const void* inv_freq, int dims, int halves, void* raw_b, int raw_ld, int dtype, hipStream_t stream) {
    TL_REQUIRE(!raw_b || raw_ld >= heads_b * dim, "head_norm_rotate: the rows of the copy are too short");
    TL_REQUIRE(tokens >= 0 && heads_a >= 0 && heads_b >= 0 && heads_a + heads_b > 0 && dim > 0 && dim <= LA_MAX_DIM && ld >= (heads_a + heads_b) * dim,
               "head_norm_rotate: bad sizes");
    TL_REQUIRE(!inv_freq || (positions && dims > 0 && dims % 2 == 0 && dims <= dim), "head_norm_rotate: a rotation over %d of %d numbers", dims, dim);
    TL_REQUIRE((norm_a == nullptr) == (norm_b == nullptr) || heads_a == 0 || heads_b == 0, "head_norm_rotate: a norm for both kinds of heads or for neither");
    if (tokens == 0) return TL_OK;
    const long items = (long)tokens * (heads_a + heads_b);
    const int grid = (int)((items + HNR_WAVES - 1) / HNR_WAVES);
    if (dtype == TL_DT_F32)
        head_norm_rotate_kernel<float><<<grid, HNR_WAVES * TL_WAVE, 0, stream>>>((float*)x, ld, tokens, heads_a, heads_b, dim, (const float*)norm_a,
            (const float*)norm_b, eps, (const int*)positions, (const float*)inv_freq, dims, halves, (float*)raw_b, raw_ld);
    else if (dtype == TL_DT_BF16)
        head_norm_rotate_kernel<bf16_t><<<grid, HNR_WAVES * TL_WAVE, 0, stream>>>((bf16_t*)x, ld, tokens, heads_a, heads_b, dim, (const float*)norm_a,
            (const float*)norm_b, eps, (const int*)positions, (const float*)inv_freq, dims, halves, (bf16_t*)raw_b, raw_ld);
    else TL_REQUIRE(false, "head_norm_rotate: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("head_norm_rotate");
    return TL_OK;
}
