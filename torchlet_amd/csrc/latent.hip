// Attention over a cached latent: every token keeps one row of `rank` normed latent numbers followed by `rot`
// rotated key numbers that all heads share.  A head's query is brought into the same shape beforehand (its
// unrotated part multiplied through the key up-projection, its rotated part turned by its position), so a
// score is one dot product of rank + rot numbers and the weighted sum runs over the latent rows themselves;
// the value up-projection follows outside.  Norms, angles, scores, weights and sums are float.
#include "common.h"

// A barrier that orders shared memory only: __syncthreads() also waits for every fetch from memory that is on its
// way (its fence covers global memory), which would end a prefetch at the first barrier after it.
__device__ __forceinline__ void shared_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The pair (u, v) at entries (2i, 2i + 1) turned by position * inv_freq[i].
__device__ __forceinline__ void turn_pair(float u, float v, float pos, float f, float& a, float& b) {
    float s, c;
    sincosf(pos * f, &s, &c);
    a = u * c - v * s;
    b = v * c + u * s;
}

// ------------------------------------------------------------------ norms of the two latents, rotation, cache write
// down [tokens, ld]: q_rank numbers of the query latent (q_rank 0: none), and from column kv_off on rank numbers of the key/value
// latent, then rot of the shared key part.
// cq = rmsnorm(first q_rank) * wq;  page row of the token = [rmsnorm(the rank numbers) * wkv, the last rot with the first
// rot_dims of them turned in pairs].  A token whose block-table entry is 0 (the sentinel page) writes nothing.
template <typename T>
__global__ void latent_prepare_kernel(const T* __restrict__ down, int ld, int q_rank, int kv_off, int rank, int rot, int rot_dims,
                                      const void* __restrict__ wq, int wq_f32, const void* __restrict__ wkv, int wkv_f32, float eps,
                                      const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                      const int* __restrict__ token_req, const int* __restrict__ block_table, int bt_stride,
                                      T* __restrict__ plane, int page_size, T* __restrict__ cq) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const T* row = down + (size_t)t * ld;
    float ss = 0.f, inv = 0.f;
    if (q_rank > 0) {
        for (int i = threadIdx.x; i < q_rank; i += blockDim.x) { const float x = to_float(row[i]); ss = fmaf(x, x, ss); }
        ss = block_sum(ss, red);
        inv = 1.f / sqrtf(ss / (float)q_rank + eps);
        for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
            cq[(size_t)t * q_rank + i] = from_float<T>(to_float(row[i]) * inv * load_vec(wq, wq_f32, i));
    }
    if (plane == nullptr) return;
    const int pos = positions[t];
    const int page = block_table[(size_t)token_req[t] * bt_stride + pos / page_size];
    ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) { const float x = to_float(row[kv_off + i]); ss = fmaf(x, x, ss); }
    ss = block_sum(ss, red);
    if (page == 0) return;
    inv = 1.f / sqrtf(ss / (float)rank + eps);
    T* dst = plane + ((size_t)page * page_size + pos % page_size) * (rank + rot);
    for (int i = threadIdx.x; i < rank; i += blockDim.x)
        dst[i] = from_float<T>(to_float(row[kv_off + i]) * inv * load_vec(wkv, wkv_f32, i));
    const T* kr = row + kv_off + rank;
    for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
        float a, b;
        turn_pair(to_float(kr[2 * i]), to_float(kr[2 * i + 1]), (float)pos, inv_freq[i], a, b);
        dst[rank + 2 * i] = from_float<T>(a);
        dst[rank + 2 * i + 1] = from_float<T>(b);
    }
    for (int i = rot_dims + threadIdx.x; i < rot; i += blockDim.x) dst[rank + i] = kr[i];
}

extern "C" int tl_latent_prepare(const void* down, int ld, int q_rank, int kv_off, int rank, int rot, int rot_dims, const void* wq, int wq_f32,
                                 const void* wkv, int wkv_f32, float eps, const void* positions, const void* inv_freq,
                                 const void* token_req, const void* block_table, int bt_stride, void* plane, int page_size,
                                 void* cq, int tokens, int dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && q_rank >= 0 && kv_off >= q_rank && rank > 0 && rot >= 0 && rot_dims % 2 == 0 && rot_dims <= rot && ld >= kv_off + rank + rot,
               "latent_prepare: bad sizes");
    TL_REQUIRE(q_rank == 0 || (wq && cq), "latent_prepare: a query latent needs its norm's weight and a place to go");
    TL_REQUIRE(plane == nullptr || (page_size > 0 && block_table != nullptr && token_req != nullptr), "latent_prepare: a cache write needs the block table");
    if (tokens == 0) return TL_OK;
    dim3 grid(tokens), block(256);
#define TL_ARGS(T) (const T*)down, ld, q_rank, kv_off, rank, rot, rot_dims, wq, wq_f32, wkv, wkv_f32, eps, (const int*)positions, (const float*)inv_freq, \
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
                        int splits, float* __restrict__ part_o, float* __restrict__ part_ml, int window, const T* __restrict__ gate, int gate_ld) {
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
    // with a window a row at qpos reads the keys qpos - window + 1 .. qpos; the tile starts at the step of LAT_KT keys (counted from
    // position 0, so that a key's step does not depend on the tile) in which its first row's first key lies
    const int tile_first = window > 0 ? max(0, ctx + tok0 - window + 1) : 0;
    const int kbegin = tile_first / LAT_KT * LAT_KT;
    const int qfirst = window > 0 ? max(0, qpos - window + 1) : 0;
    for (int k0 = kbegin + split * LAT_KT; k0 <= last; k0 += splits * LAT_KT) {
        __syncthreads();
        const int nk = min(LAT_KT, last + 1 - k0);
        for (int i = threadIdx.x; i < nk * D; i += blockDim.x) {
            const int kk = i / D, d = i % D, pos = k0 + kk;
            const int page = table[pos / page_size];
            // (what lies before the tile's first key may be gone with its page: it counts as zeros)
            sk[kk * ldk + d] = pos >= tile_first ? to_float(plane[((size_t)page * page_size + pos % page_size) * D + d]) : 0.f;
        }
        __syncthreads();
        if (!row_ok || k0 > qpos || k0 + nk <= qfirst) continue;
        // scores: lanes 0..KT-1 take one key each (the upper half of the wave idles here)
        float s = -INFINITY;
        if (lane < nk && k0 + lane <= qpos && k0 + lane >= qfirst) {
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
        float inv = l > 0.f ? 1.f / l : 0.f;
        if (gate) inv *= 1.f / (1.f + expf(-to_float(gate[(size_t)tok * gate_ld + rh])));
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
// The parts' weights are worked out once per row (by the first threads, into shared memory), then every thread sums its
// columns, neighbours reading neighbouring numbers.
#define LAT_MAX_SPLITS 64
template <typename T>
__global__ void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, T* __restrict__ out,
                                    int rows, int rank, int splits, const T* __restrict__ gate, int gate_ld, int heads) {
    __shared__ float wgt[LAT_MAX_SPLITS];
    __shared__ float inv_s;
    const int row = blockIdx.x;
    const float* ml = part_ml + (size_t)row * splits * 2;
    if (threadIdx.x < TL_WAVE) {
        const int s = threadIdx.x;
        const float ms = s < splits ? ml[s * 2] : -INFINITY;
        const float M = wave_max(ms);
        const float w = (s < splits && ms != -INFINITY) ? expf(ms - M) : 0.f;
        if (s < splits) wgt[s] = w;
        float den = 0.f;
        for (int i = 0; i < splits; ++i) {             // in the order of the parts
            const float wi = __shfl(w, i, TL_WAVE), li = ml[i * 2 + 1];
            den += wi * li;
        }
        if (s == 0) {
            float inv0 = den > 0.f ? 1.f / den : 0.f;
            if (gate) inv0 *= 1.f / (1.f + expf(-to_float(gate[(size_t)(row / heads) * gate_ld + row % heads])));
            inv_s = inv0;
        }
    }
    __syncthreads();
    const float inv = inv_s;
    const float* po = part_o + (size_t)row * splits * rank;
    for (int c = threadIdx.x; c < rank; c += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < splits; ++s) a = fmaf(wgt[s], po[(size_t)s * rank + c], a);
        out[(size_t)row * rank + c] = from_float<T>(a * inv);
    }
}

// ------------------------------------------------------------------ attention on the matrix cores (bfloat16)
// The same attention with both products on v_mfma_f32_16x16x32_bf16, transposed so that no result changes layout on its
// way into the next product: S^T = K Q^T (a lane holds four keys of one query), O^T = L^T P^T (L the latent part of the
// cached rows).  The first product sums over a row's numbers, which lie side by side in the cache; the second sums over
// keys, so it wants the latents of neighbouring keys side by side: a step's 32 rows go to shared memory twice, as they
// lie in the cache and transposed, written there once by the whole work-group.
// A work-group of four waves owns RB blocks of 16 rows (row = token x head of a chunk of up to 16 heads; RB = 4, 2 or 1
// by how many rows a tile of the step can have) and 4 / RB waves share a block: each takes all of the block's scores
// (the softmax's state is then the same in all of them, nothing is exchanged) and its own share of the latent's columns.
#define LM_KEYS 32                    // keys of a step
#define LM_DC_MAX 20                  // 32-number pieces of a cache row (rows of up to 640 numbers)
#define LM_LOG2E 1.4426950408889634f
#define LM_BT_MAX 1536                // block-table entries of a request that a work-group keeps in shared memory (two work-groups fit a compute unit)

typedef __bf16 lm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lm_f32x4 __attribute__((ext_vector_type(4)));
union LmFrag {
    uint4 u;
    uint2 h[2];
    lm_bf16x8 v;
};

template <int RB>
__global__ void __launch_bounds__(256)
latent_attention_mfma_kernel(const bf16_t* __restrict__ q, int q_ld, bf16_t* __restrict__ out, const bf16_t* __restrict__ plane,
                             const int* __restrict__ block_table, int bt_stride, const int* __restrict__ req_indptr,
                             const int* __restrict__ ctx_lens, const int* __restrict__ tile_req, const int* __restrict__ tile_tok0,
                             int tile_tokens, int heads, int rank, int rot, int page_size, float scale, const float* __restrict__ sink,
                             int splits, float* __restrict__ part_o, float* __restrict__ part_ml, int window, const bf16_t* __restrict__ gate,
                             int gate_ld) {
    constexpr int WPR = 4 / RB;                      // waves that share a block of rows
    constexpr int NT = 32 / WPR;                     // most blocks of 16 latent columns a wave sums (latents of up to 512 numbers)
    extern __shared__ __align__(16) unsigned char lm_smem[];
    const int D = rank + rot, dc = D / 32, ldk = D + 8, ldt = LM_KEYS + 4;
    bf16_t* sk = (bf16_t*)lm_smem;                   // [32 keys][D + 8]: rows as they lie in the cache
    bf16_t* st = sk + LM_KEYS * ldk;                 // [rank][32 + 4]: the latents transposed
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, g = lane >> 4;
    const int rb = wave / WPR, share = wave % WPR;
    const int tile = blockIdx.x, head0 = blockIdx.y * 16, split = blockIdx.z;
    const int hchunk = min(16, heads - head0);
    const int req = tile_req ? tile_req[tile] : tile, tok0 = tile_req ? tile_tok0[tile] : 0;
    const int first = req_indptr ? req_indptr[req] : req, n_new = req_indptr ? req_indptr[req + 1] - first : 1;
    const int ctx = ctx_lens[req];
    const int ntok = min(tile_tokens, n_new - tok0);
    const int rows = ntok * hchunk;
    // the query this lane's column of S^T belongs to
    const int row = rb * 16 + li;
    const bool row_ok = row < rows;
    const int rt = row_ok ? row / hchunk : 0, rh = head0 + (row_ok ? row % hchunk : 0);
    const int tok = first + tok0 + rt, qpos = ctx + tok0 + rt;
    const int qfirst = window > 0 ? max(0, qpos - window + 1) : 0;      // the first key this query reads
    const int tile_first = window > 0 ? max(0, ctx + tok0 - window + 1) : 0;      // ... and the first one any query of the tile reads
    LmFrag qf[LM_DC_MAX];
#pragma unroll
    for (int c = 0; c < LM_DC_MAX; ++c)
        qf[c].u = (c < dc && row_ok) ? *(const uint4*)(q + (size_t)tok * q_ld + (size_t)rh * D + 32 * c + 8 * g) : make_uint4(0, 0, 0, 0);
    const int nt = rank / 16 / WPR;                  // blocks of 16 latent columns of this wave: t0 .. t0 + nt - 1
    const int t0 = share * nt;
    lm_f32x4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = lm_f32x4{0.f, 0.f, 0.f, 0.f};
    const bool with_sink = sink != nullptr && split == 0;
    float m = with_sink ? sink[rh] * LM_LOG2E : -INFINITY;      // base 2: scores are taken times scale * log2(e)
    float l = (with_sink && g == 0) ? 1.f : 0.f;                // (a lane sums its own keys; the lanes of a query are added at the end)
    const float scale2 = scale * LM_LOG2E;
    const int last = ctx + tok0 + ntok - 1;
    const int* table = block_table + (size_t)req * bt_stride;
    // A step's 32 rows come through registers: a wave brings 8 of them, lane (key = lane % 8, piece = lane / 8 + 8 i) a
    // 16-byte piece per round i, so that the lanes that write the transposed copy lie side by side along the keys: two
    // neighbouring lanes (an even key and the next) swap halves of their pieces and each writes four 32-bit words that hold
    // both keys' numbers of one column.  The rows of the step after are requested before this step's products start and
    // written when they are done.
    const int pieces = D / 8, rounds = (pieces + 7) / 8;
    const int kk = wave * 8 + (lane & 7), pg = lane >> 3;       // the key of the step that this lane brings, and its piece of a round
    const bool odd = lane & 1;
    // The request's block-table row lies in shared memory (the host sees to it that it fits): a step's rows are then one
    // trip to memory, and, more to the point, looking a page up does not wait on the memory counter, which counts in order:
    // a wait for a table entry would be a wait for every row requested before it, the rows of the steps ahead included.
    int* tbl = (int*)(st + (size_t)rank * ldt);
    for (int i = threadIdx.x; i <= last / page_size; i += 256) tbl[i] = table[i];
    __syncthreads();
    constexpr bool TWO = RB < 4;                     // steps requested ahead: two where the registers allow it
    const int stride = splits * LM_KEYS, ahead = TWO ? 2 * stride : stride;
    uint4 stage0[LM_DC_MAX / 2], stage1[TWO ? LM_DC_MAX / 2 : 1];
    // where this lane's pieces go in shared memory does not change from step to step
    bf16_t* const sk_mine = sk + kk * ldk + 8 * pg;
    uint32_t* const st_mine = (uint32_t*)(st + (8 * pg + (odd ? 4 : 0)) * ldt + (kk & ~1));
    const int page_shift = (page_size & (page_size - 1)) == 0 ? __ffs(page_size) - 1 : -1;
    // (every lane fetches, from a clamped place where its own lies beyond the keys or the row: a fetch under a condition
    // would be waited for on the spot; what must be zero is cleared when the pieces are written to shared memory)
    auto request = [&](uint4 (&stage)[LM_DC_MAX / 2], int at) {
        const int pos = max(min(at + kk, last), tile_first);
        const int blk = page_shift >= 0 ? pos >> page_shift : pos / page_size;
        const bf16_t* src = plane + ((size_t)tbl[blk] * page_size + (pos - blk * page_size)) * D;
#pragma unroll
        for (int i = 0; i < LM_DC_MAX / 2; ++i)
            if (i < rounds) stage[i] = *(const uint4*)(src + 8 * min(pg + 8 * i, pieces - 1));
    };
    auto step = [&](uint4 (&stage)[LM_DC_MAX / 2], int k0) {
        shared_barrier();                             // the products of the step before have read shared memory
#pragma unroll
        for (int i = 0; i < LM_DC_MAX / 2; ++i) {
            if (i < rounds) {
                const int col = 64 * i + 8 * pg;
                const uint4 x = (k0 + kk <= last && k0 + kk >= tile_first && col < D) ? stage[i] : make_uint4(0, 0, 0, 0);
                // the neighbour's half: the even lane keeps its first four numbers and gets the neighbour's, the odd lane the last four
                const uint32_t mine0 = odd ? x.z : x.x, mine1 = odd ? x.w : x.y;
                const uint32_t got0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)(odd ? x.x : x.z), 0xB1, 0xF, 0xF, true);
                const uint32_t got1 = (uint32_t)__builtin_amdgcn_mov_dpp((int)(odd ? x.y : x.w), 0xB1, 0xF, 0xF, true);
                if (col < D) {
                    *(uint4*)(sk_mine + 64 * i) = x;
                    if (col < rank) {
                        const uint32_t a0 = odd ? got0 : mine0, b0 = odd ? mine0 : got0;      // (even key, odd key)
                        const uint32_t a1 = odd ? got1 : mine1, b1 = odd ? mine1 : got1;
                        uint32_t* dst = st_mine + 32 * i * ldt;
                        dst[0] = (a0 & 0xffffu) | (b0 << 16);
                        dst[ldt / 2] = (a0 >> 16) | (b0 & 0xffff0000u);
                        dst[ldt] = (a1 & 0xffffu) | (b1 << 16);
                        dst[3 * (ldt / 2)] = (a1 >> 16) | (b1 & 0xffff0000u);
                    }
                }
            }
        }
        shared_barrier();
        if (k0 + ahead <= last) request(stage, k0 + ahead);
#pragma unroll
        for (int j = 0; j < LM_KEYS / 32; ++j) {
            const int kbase = k0 + 32 * j;
            // ---- scores of 32 keys, as two halves of 16
            float sc[8];
            {
                // four chains of products (two halves of keys, the pieces of a row dealt to two sums each): a product that
                // adds to the one before it waits for it
                lm_f32x4 s00 = lm_f32x4{0.f, 0.f, 0.f, 0.f}, s01 = s00, s10 = s00, s11 = s00;
                const bf16_t* krow0 = sk + (32 * j + li) * ldk + 8 * g;
                const bf16_t* krow1 = krow0 + 16 * ldk;
#pragma unroll
                for (int c = 0; c < LM_DC_MAX; c += 2) {
                    if (c < dc) {
                        LmFrag k0f, k1f;
                        k0f.u = *(const uint4*)(krow0 + 32 * c);
                        k1f.u = *(const uint4*)(krow1 + 32 * c);
                        s00 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0f.v, qf[c].v, s00, 0, 0, 0);
                        s10 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1f.v, qf[c].v, s10, 0, 0, 0);
                    }
                    if (c + 1 < dc) {
                        LmFrag k0f, k1f;
                        k0f.u = *(const uint4*)(krow0 + 32 * (c + 1));
                        k1f.u = *(const uint4*)(krow1 + 32 * (c + 1));
                        s01 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0f.v, qf[c + 1].v, s01, 0, 0, 0);
                        s11 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1f.v, qf[c + 1].v, s11, 0, 0, 0);
                    }
                }
                s00 += s01;
                s10 += s11;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = kbase + 4 * g + v;
                    sc[v] = (row_ok && key <= qpos && key >= qfirst) ? s00[v] * scale2 : -INFINITY;
                    sc[4 + v] = (row_ok && key + 16 <= qpos && key + 16 >= qfirst) ? s10[v] * scale2 : -INFINITY;
                }
            }
            float mloc = sc[0];
#pragma unroll
            for (int i = 1; i < 8; ++i) mloc = fmaxf(mloc, sc[i]);
            mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
            const float m_new = fmaxf(m, mloc);
            const float alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);     // (m_new may still be -inf: a step wholly before this query's window)
            const bool moved = __any(m_new != m);    // the sums are rescaled only when some query's maximum moved
            LmFrag pf;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = (sc[i] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sc[i] - m_new);
                psum += p;
                pf.v[i] = (__bf16)p;
            }
            l = l * alpha + psum;
            m = m_new;
            // ---- O^T += L^T P^T over this wave's share of the latent's columns
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (t < nt) {
                    const bf16_t* lrow = st + (16 * (t0 + t) + li) * ldt + 32 * j + 4 * g;
                    LmFrag vf;
                    vf.h[0] = *(const uint2*)lrow;
                    vf.h[1] = *(const uint2*)(lrow + 16);
                    if (moved) acc[t] *= alpha;
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, acc[t], 0, 0, 0);
                }
            }
        }
    };
    // (with a window the tile starts at the step, counted from position 0, in which its first token's first key lies)
    const int kfirst = tile_first / LM_KEYS * LM_KEYS + split * LM_KEYS;
    if (kfirst <= last) request(stage0, kfirst);
    if constexpr (TWO) {
        if (kfirst + stride <= last) request(stage1, kfirst + stride);
        for (int k0 = kfirst; k0 <= last; k0 += 2 * stride) {
            step(stage0, k0);
            if (k0 + stride <= last) step(stage1, k0 + stride);
        }
    } else {
        for (int k0 = kfirst; k0 <= last; k0 += stride) step(stage0, k0);
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!row_ok) return;
    if (splits == 1) {
        float inv = l > 0.f ? 1.f / l : 0.f;
        if (gate) inv *= 1.f / (1.f + expf(-to_float(gate[(size_t)tok * gate_ld + rh])));
        bf16_t* o = out + ((size_t)tok * heads + rh) * rank;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t < nt) {
                union { uint2 u; uint16_t e[4]; } pk;
#pragma unroll
                for (int v = 0; v < 4; ++v) pk.e[v] = from_float<bf16_t>(acc[t][v] * inv).bits;
                *(uint2*)(o + 16 * (t0 + t) + 4 * g) = pk.u;
            }
        }
    } else {
        const size_t prow = ((size_t)tok * heads + rh) * splits + split;
        float* o = part_o + prow * rank;
#pragma unroll
        for (int t = 0; t < NT; ++t)
            if (t < nt) *(lm_f32x4*)(o + 16 * (t0 + t) + 4 * g) = acc[t];
        if (share == 0 && g == 0) { part_ml[prow * 2] = m / LM_LOG2E; part_ml[prow * 2 + 1] = l; }       // the merge works in base e
    }
}

static size_t lm_smem_bytes(int rank, int rot) { return sizeof(bf16_t) * ((size_t)LM_KEYS * (rank + rot + 8) + (size_t)rank * (LM_KEYS + 4)) + sizeof(int) * LM_BT_MAX; }

// Whether the matrix-core kernel is built for these sizes: rows of a multiple of 32 numbers up to 640, latents of a
// multiple of 64 numbers up to 512, 16-byte aligned query rows.
static bool lm_fits(int rank, int rot, int q_ld, const void* q, const void* plane, int bt_stride) {
    const int D = rank + rot;
    return bt_stride <= LM_BT_MAX && D % 32 == 0 && D <= 32 * LM_DC_MAX && rank % 64 == 0 && rank <= 512 && q_ld % 8 == 0 &&
           ((uintptr_t)q % 16) == 0 && ((uintptr_t)plane % 16) == 0 && lm_smem_bytes(rank, rot) <= 160 * 1024;
}

template <int RB>
static int launch_lm(const void* q, int q_ld, void* out, const void* plane, const void* block_table, int bt_stride, const void* req_indptr,
                     const void* ctx_lens, const void* tile_req, const void* tile_tok0, int num_tiles, int tile_tokens, int heads, int rank,
                     int rot, int page_size, float scale, const void* sink, int splits, void* part_o, void* part_ml, int window, const void* gate,
                     int gate_ld, hipStream_t stream) {
    static size_t allowed = 48 * 1024;               // (per instance of the template)
    const size_t smem = lm_smem_bytes(rank, rot);
    auto kernel = latent_attention_mfma_kernel<RB>;
    if (smem > allowed) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
            tl_set_error("latent_attention: cannot get %zu bytes of shared memory", smem); return TL_ERR_HIP;
        }
        allowed = smem;
    }
    dim3 grid(num_tiles, (heads + 15) / 16, splits), block(256);
    kernel<<<grid, block, smem, stream>>>((const bf16_t*)q, q_ld, (bf16_t*)out, (const bf16_t*)plane, (const int*)block_table, bt_stride,
                                          (const int*)req_indptr, (const int*)ctx_lens, (const int*)tile_req, (const int*)tile_tok0, tile_tokens,
                                          heads, rank, rot, page_size, scale, (const float*)sink, splits, (float*)part_o, (float*)part_ml, window,
                                          (const bf16_t*)gate, gate_ld);
    TL_CHECK_LAUNCH("latent_attention_mfma");
    return TL_OK;
}

extern "C" int tl_latent_attention_mfma_fits(int rank, int rot, int q_ld) {
    const int D = rank + rot;
    return (D % 32 == 0 && D <= 32 * LM_DC_MAX && rank % 64 == 0 && rank <= 512 && q_ld % 8 == 0 && lm_smem_bytes(rank, rot) <= 160 * 1024) ? 1 : 0;
}

// q [tokens, q_ld]: per head rank + rot numbers (head h at column h * (rank + rot)); out [tokens, heads * rank];
// plane [pages, page_size, rank + rot]; sink float [heads] or null; tile_req null: tile i is the one token of request i.
// window > 0: a query reads its last `window` keys only, itself included.  gate (of the activation type, [tokens, gate_ld], or null):
// head h's output of token t is multiplied by sigmoid(gate[t, h]).
extern "C" int tl_latent_attention(const void* q, int q_ld, void* out, const void* plane, const void* block_table, int bt_stride,
                                   const void* req_indptr, const void* ctx_lens, const void* tile_req, const void* tile_tok0,
                                   int num_tiles, int tokens, int tile_tokens, int heads, int rank, int rot, int page_size, float scale,
                                   const void* sink, int splits, void* part_o, void* part_ml, int dtype, int general, int max_new_tokens,
                                   int window, const void* gate, int gate_ld, hipStream_t stream) {
    TL_REQUIRE(window >= 0 && (!gate || gate_ld >= heads), "latent_attention: a window is not negative and a gate has a number per head");
    TL_REQUIRE(num_tiles >= 0 && heads > 0 && rank > 0 && rot >= 0 && page_size > 0 && tile_tokens > 0, "latent_attention: bad sizes");
    TL_REQUIRE(rank <= 16 * TL_WAVE, "latent_attention: built for latents of up to %d numbers, got %d", 16 * TL_WAVE, rank);
    TL_REQUIRE(splits >= 1 && splits <= LAT_MAX_SPLITS && (splits == 1 || (part_o != nullptr && part_ml != nullptr)), "latent_attention: 1 to 64 parts, with their scratch");
    TL_REQUIRE(q_ld >= heads * (rank + rot), "latent_attention: query rows are too short");
    if (num_tiles == 0) return TL_OK;
    const int tile_rows = min(tile_tokens, max(1, max_new_tokens)) * min(heads, 16);       // most rows a tile of this step has
    if (dtype == TL_DT_BF16 && !general && lm_fits(rank, rot, q_ld, q, plane, bt_stride)) {
        TL_REQUIRE(tile_tokens * min(heads, 16) <= 64, "latent_attention: a tile of %d tokens and %d heads has more than 64 rows", tile_tokens, heads);
        int rc;
#define TL_LM(RB) rc = launch_lm<RB>(q, q_ld, out, plane, block_table, bt_stride, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles, tile_tokens, \
                                     heads, rank, rot, page_size, scale, sink, splits, part_o, part_ml, window, gate, gate_ld, stream)
        if (tile_rows <= 16) TL_LM(1); else if (tile_rows <= 32) TL_LM(2); else TL_LM(4);
#undef TL_LM
        if (rc != TL_OK) return rc;
        if (splits > 1) {
            const int rows = tokens * heads;
            latent_merge_kernel<bf16_t><<<rows, 128, 0, stream>>>((const float*)part_o, (const float*)part_ml, (bf16_t*)out, rows, rank, splits,
                                                                  (const bf16_t*)gate, gate_ld, heads);
            TL_CHECK_LAUNCH("latent_merge");
        }
        return TL_OK;
    }
    TL_REQUIRE(tile_tokens * min(heads, LAT_ROWS) <= LAT_ROWS, "latent_attention: a tile of %d tokens and %d heads has more than %d rows", tile_tokens, heads, LAT_ROWS);
    const int D = rank + rot;
    const size_t smem = sizeof(float) * ((size_t)LAT_KT * (D + 1) + (size_t)LAT_ROWS * D + LAT_ROWS * LAT_KT);
    TL_REQUIRE(smem <= 160 * 1024, "latent_attention: %zu bytes of shared memory for rows of %d numbers", smem, D);
    dim3 grid(num_tiles, (heads + LAT_ROWS - 1) / LAT_ROWS, splits), block(LAT_ROWS * TL_WAVE);
#define TL_ARGS(T) (const T*)q, q_ld, (T*)out, (const T*)plane, (const int*)block_table, bt_stride, (const int*)req_indptr, (const int*)ctx_lens, \
                   (const int*)tile_req, (const int*)tile_tok0, tile_tokens, heads, rank, rot, page_size, scale, (const float*)sink, splits,      \
                   (float*)part_o, (float*)part_ml, window, (const T*)gate, gate_ld
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
        if (dtype == TL_DT_F32) latent_merge_kernel<float><<<rows, 128, 0, stream>>>((const float*)part_o, (const float*)part_ml, (float*)out, rows, rank, splits,
                                                                                     (const float*)gate, gate_ld, heads);
        else latent_merge_kernel<bf16_t><<<rows, 128, 0, stream>>>((const float*)part_o, (const float*)part_ml, (bf16_t*)out, rows, rank, splits,
                                                                   (const bf16_t*)gate, gate_ld, heads);
        TL_CHECK_LAUNCH("latent_merge");
    }
    return TL_OK;
}
