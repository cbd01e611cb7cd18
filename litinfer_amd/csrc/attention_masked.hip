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

// Orders a wave's own LDS writes before its own later LDS reads (other lanes' data included: a wave's LDS
// instructions are carried out in the order of their issue), without the block's barrier.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// What a (token, head)'s sums of values are multiplied by at the end: one over the sum of the weights, to which a
// softmax with a SINK adds exp(sink[head] - maximum) (a term of the denominator that has no key and no value), and,
// where the heads have gates, times sigmoid(gate[token, head]).
__device__ __forceinline__ float finish_factor(float l, float m, const float* __restrict__ sink, const float* __restrict__ gate,
                                               long gate_stride, int t, int head) {
    if (sink && l != 0.f) l += expf(sink[head] - m);
    float f = l != 0.f ? 1.0f / l : 0.f;
    if (gate) f *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_stride + head]));
    return f;
}

// The general kernel (any sizes, both dtypes): a block of NW waves per (token, query head); wave w takes the
// rounds w, w + NW, ... of 64 visible keys.  In a round a lane takes one key for the scores (its row read in
// 16-byte pieces where the rows allow it), then one value column (and every 64th after it) for the sums.  The
// waves' running (maximum, sum, sums of values) are joined through LDS in wave order.
template <typename T, typename TO, int NC, bool VEC, int NW>
__global__ __launch_bounds__(64 * NW) void masked_attention_wave_kernel(
    const float* __restrict__ q, int q_token_stride, int q_head_stride, TO* __restrict__ out,
    const T* __restrict__ kc, const T* __restrict__ vc, int k_row, int v_row,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_list,
    const int* __restrict__ seg_of_token,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    int nh, int nkv, int dk, int dv, int page_size, int num_pages, int window, int keep_first, float softcap, float scale, const float* __restrict__ sink, const float* __restrict__ gate, long gate_stride) {
    extern __shared__ float smem[];
    float* qs = smem;                                        // [dk]
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    float* ps = smem + dk + w * 128;                         // [64] a wave
    int* rowoff = (int*)(ps + LI_WAVE);                      // [64] a wave
    float* join = smem + dk + NW * 128;                      // [NW][dv + 2]
    const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, h = blockIdx.y;
    const int s = seg_of_token[t];
    const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_first = keep_first < lo ? keep_first : lo;
    const int n_keys = n_first + (p - lo + 1);
    const int kvh = h / (nh / nkv);
    const int* table = block_table + (size_t)s * max_blocks;
    const float* qrow = q + (size_t)t * q_token_stride + (size_t)h * q_head_stride;
    for (int d = threadIdx.x; d < dk; d += 64 * NW) qs[d] = qrow[d];
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.f;
    for (int i0 = 64 * w; i0 < n_keys; i0 += 64 * NW) {
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
        ps[lane] = e;                            // (a wave's own LDS traffic is ordered: the reads below follow these writes)
        rowoff[lane] = ro;
        wave_lds_sync();
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
        wave_lds_sync();                         // (the next round's writes follow these reads)
        m = m_new;
    }
    TO* orow = out + ((size_t)t * nh + h) * dv;
    if constexpr (NW == 1) {
        const float fin = finish_factor(l, m, sink, gate, gate_stride, t, h);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int d = lane + c * LI_WAVE;
            if (d < dv) store_from_float(orow + d, acc[c] * fin);
        }
    } else {
        float* mine = join + (size_t)w * (dv + 2);
        if (lane == 0) { mine[dv] = m; mine[dv + 1] = l; }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int d = lane + c * LI_WAVE;
            if (d < dv) mine[d] = acc[c];
        }
        __syncthreads();
        float mm = -INFINITY;
        for (int x = 0; x < NW; ++x) mm = fmaxf(mm, join[(size_t)x * (dv + 2) + dv]);
        float ll = 0.f;
        float f[NW];
#pragma unroll
        for (int x = 0; x < NW; ++x) {
            const float mx = join[(size_t)x * (dv + 2) + dv], lx = join[(size_t)x * (dv + 2) + dv + 1];
            f[x] = (lx == 0.f) ? 0.f : expf(mx - mm);
            ll += lx * f[x];
        }
        const float fin = finish_factor(ll, mm, sink, gate, gate_stride, t, h);
        for (int d = threadIdx.x; d < dv; d += 64 * NW) {
            float a = 0.f;
#pragma unroll
            for (int x = 0; x < NW; ++x) a += join[(size_t)x * (dv + 2) + d] * f[x];
            store_from_float(orow + d, a * fin);
        }
    }
}

template <typename T, typename TO, int NC>
static int launch_masked(const float* q, int qts, int qhs, void* out, const void* kc, const void* vc, int k_row, int v_row,
                         const int* block_table, int max_blocks, const int* token_list, int n_tokens, const int* seg_of_token,
                         const int* q_start, const int* q_len,
                         const int* ctx_len, int nh, int nkv, int dk, int dv, int page_size, int num_pages, int window,
                         int keep_first, float softcap, float scale, const float* sink, const float* gate, long gate_stride, int waves, hipStream_t stream) {
    const dim3 grid(n_tokens, nh);
    constexpr int E = 16 / sizeof(T);
    const bool vec = dk % E == 0 && k_row % E == 0 && ((uintptr_t)kc % 16) == 0;
#define MA_GO(V, NW)                                                                                                         \
    masked_attention_wave_kernel<T, TO, NC, V, NW><<<grid, 64 * NW, (size_t)(dk + NW * 128 + NW * (dv + 2)) * 4, stream>>>(  \
        q, qts, qhs, (TO*)out, (const T*)kc, (const T*)vc, k_row, v_row, block_table, max_blocks, token_list, seg_of_token,  \
        q_start, q_len, ctx_len, nh, nkv, dk, dv, page_size, num_pages, window, keep_first, softcap, scale, sink, gate, gate_stride)
    if (waves >= 8) { if (vec) MA_GO(true, 8); else MA_GO(false, 8); }
    else if (waves >= 4) { if (vec) MA_GO(true, 4); else MA_GO(false, 4); }
    else { if (vec) MA_GO(true, 1); else MA_GO(false, 1); }
#undef MA_GO
    return li_launch_status();
}

// q float32: head h of token t at q + t * q_token_stride + h * q_head_stride (dk values).  out [T, nh, dv] of
// out_dtype.  kc / vc: rows of k_row / v_row elements of cache_dtype, row (page * nkv + kv head) * page_size + place;
// the key is the first dk and the value the first dv elements of its row (the two may be the same memory).
// token_list (or null: tokens 0 .. n_tokens - 1): the tokens this call takes.  waves: 1, 4 or 8 waves share a
// (token, head)'s keys.
extern "C" int li_masked_attention(const float* q, int q_token_stride, int q_head_stride, void* out, int out_dtype,
                                   const void* kc, const void* vc, int cache_dtype, int k_row, int v_row,
                                   const int* block_table, int max_blocks, const int* token_list, int n_tokens,
                                   const int* seg_of_token, const int* q_start,
                                   const int* q_len, const int* ctx_len, int nh, int nkv, int dk, int dv,
                                   int page_size, int num_pages, int window, int keep_first, float softcap, float scale, const float* sink, const float* gate, long gate_stride,
                                   int waves, hipStream_t stream) {
    if (n_tokens <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dv <= 0 || dk > k_row || dv > v_row || page_size <= 0 ||
        window < 0 || keep_first < 0 || max_blocks <= 0 || nh > 65535 || dk > 4096 || dv > 64 * MA_MAX_CHUNKS)
        return LI_ERR_SIZE;
    const int nc = (dv + 63) / 64;
#define MA_ARGS q, q_token_stride, q_head_stride, out, kc, vc, k_row, v_row, block_table, max_blocks, token_list, n_tokens,  \
                seg_of_token, q_start, q_len, ctx_len, nh, nkv, dk, dv, page_size, num_pages, window, keep_first, softcap,   \
                scale, sink, gate, gate_stride, waves, stream
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

// ------------------------------------------------------------------------------------------- tiles of queries, MFMA
// Portions of prompts in bfloat16: a block takes a tile of up to 32 consecutive queries of one request and one kv
// head; its (up to four) waves are query heads of that kv head and share every block of 32 keys and values, which
// the block stages in LDS.  A wave works on the TRANSPOSED scores S^T[key, query] = K Q^T (v_mfma_f32_32x32x16_bf16;
// row operand K from LDS, column operand Q in registers as bfloat16): a lane then holds 16 keys of ITS query
// (register r: key 8 (r / 4) + 4 (l / 32) + r % 4), so scale, cap, mask and softmax are arithmetic inside a lane plus
// one exchange with lane l ^ 32, and the probabilities, rounded to bfloat16, are the column operand of
// O^T[d, query] = V^T P^T as they are.  Its row operand V^T wants, for one value column, the keys
// {16 s + 4 h + i, 16 s + 8 + 4 h + i : i < 4} side by side: the values are written to LDS transposed and in that
// order.  The visible keys of a tile are its kept first positions and the window of its first to its last query;
// they are walked as one list (`visible_key`), 32 at a time.
// exponential and tanh by the hardware's exp2 and reciprocal (relative error about 2^-22: the bfloat16 kernels
// round their probabilities to 8 bits anyway; the float32 path keeps expf and tanhf)
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_tanh(float x) {
    const float e = __builtin_amdgcn_exp2f(fminf(x, 40.f) * 2.8853900817779268f);        // exp(2x)
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

typedef __bf16 ma_bf16x8 __attribute__((ext_vector_type(8)));
typedef float ma_f32x16 __attribute__((ext_vector_type(16)));
union ma_frag8 { uint4 raw; uint32_t w[4]; ma_bf16x8 v; };
#define MT_WAVES 4
#define MT_VS 40                    // row stride of the transposed values: 32 key places and a pad that spreads the banks

template <int KS, int DT, int NW>   // KS = dk / 16, DT = dv / 32, NW waves = heads of the kv head a block
__global__ __launch_bounds__(NW * 64) void masked_attention_tile_kernel(
    const float* __restrict__ q, int q_token_stride, int q_head_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc, int k_row, int v_row,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tiles,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    int nh, int nkv, int page_size, int num_pages, int window, int keep_first, float softcap, float scale, const float* __restrict__ sink, const float* __restrict__ gate, long gate_stride,
    int nsplit, float* __restrict__ parts) {
    constexpr int DK = KS * 16, DV = DT * 32, KROW = DK + 8;
    constexpr int NT = NW * 64;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[32 * KROW];       // [key place][dimension]
    __shared__ __attribute__((aligned(16))) uint16_t Vt[DV * MT_VS];      // [value column][key place, permuted]
    __shared__ int rows[4][32];                                           // the cache row of each key place of four blocks in turn, -1: none
    const int tile = blockIdx.x, kvh = blockIdx.y;
    const int s = tiles[4 * tile], t0 = tiles[4 * tile + 1], ntok = tiles[4 * tile + 2];
    const int p0 = ctx_len[s] - q_len[s] + (t0 - q_start[s]);             // position of the tile's first query
    const int p_last = p0 + ntok - 1;
    const int lo_min = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    const int n_first = keep_first < lo_min ? keep_first : lo_min;
    const int n_keys = n_first + (p_last - lo_min + 1);
    const int* table = block_table + (size_t)s * max_blocks;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, ql = lane & 31, h = lane >> 5;
    const int rep = nh / nkv;
    const int sp = blockIdx.z % nsplit;                                    // this block's share of the tile's blocks of keys
    const int hh = (blockIdx.z / nsplit) * NW + w;                             // this wave's head within the group
    const bool active = hh < rep;
    const int head = kvh * rep + (active ? hh : 0);
    const int pq = p0 + ql;                                               // this lane's query (ql >= ntok: none)
    const int lq = (window > 0) ? pq - window + 1 : 0;
    const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;

    ma_frag8 qf[KS];
    {
        const float* qrow = q + (size_t)(t0 + (ql < ntok ? ql : 0)) * q_token_stride + (size_t)head * q_head_stride;
#pragma unroll
        for (int st = 0; st < KS; ++st) {
            const float4 a = *reinterpret_cast<const float4*>(qrow + 16 * st + 8 * h);
            const float4 b = *reinterpret_cast<const float4*>(qrow + 16 * st + 8 * h + 4);
            qf[st].w[0] = pack2_bf16(a.x, a.y); qf[st].w[1] = pack2_bf16(a.z, a.w);
            qf[st].w[2] = pack2_bf16(b.x, b.y); qf[st].w[3] = pack2_bf16(b.z, b.w);
        }
    }
    ma_f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;
    const int lq_last = (window > 0) ? p_last - window + 1 : 0;           // the highest lower edge among the tile's queries

    // The cache row of key place tid of the block of keys that starts at list index i0 (threads 0..31).
    auto row_of = [&](int i0) -> int {
        const int i = i0 + (int)threadIdx.x;
        if (i >= n_keys) return -1;
        const int key = visible_key(i, n_first, lo_min);
        const int page = table[key / page_size];
        return (page >= 0 && page < num_pages) ? (page * nkv + kvh) * page_size + key % page_size : -1;
    };
    constexpr int NKC = (32 * (DK / 8) + NT - 1) / NT, NVC = (32 * (DV / 8) + NT - 1) / NT;
    uint4 kregA[NKC], vregA[NVC], kregB[NKC], vregB[NVC];           // two blocks of keys on their way at a time
    // a block's keys and values on their way: from memory into registers (a place without a row reads row 0 and
    // is zeroed when it is stored) ...
#define MT_LOAD(RB, kreg, vreg)                                                                                                   \
    _Pragma("unroll") for (int n = 0; n < NKC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        const int kk = (i / (DK / 8)) & 31, c = i % (DK / 8), ro = rows[RB][kk];                                      \
        kreg[n] = *reinterpret_cast<const uint4*>(kc + (size_t)(ro >= 0 ? ro : 0) * k_row + 8 * c);                   \
    }                                                                                                                 \
    _Pragma("unroll") for (int n = 0; n < NVC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        const int kk = i % 32, c = (i / 32) % (DV / 8), ro = rows[RB][kk];                                            \
        vreg[n] = *reinterpret_cast<const uint4*>(vc + (size_t)(ro >= 0 ? ro : 0) * v_row + 8 * c);                   \
    }
    // ... and from the registers into LDS: keys as they are, values transposed and in the operand's key order
#define MT_STORE(RB, kreg, vreg)                                                                                                  \
    _Pragma("unroll") for (int n = 0; n < NKC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        if (i < 32 * (DK / 8)) {                                                                                      \
            const int kk = i / (DK / 8), c = i % (DK / 8);                                                            \
            *reinterpret_cast<uint4*>(&Ks[kk * KROW + 8 * c]) = rows[RB][kk] >= 0 ? kreg[n] : uint4{0u, 0u, 0u, 0u};  \
        }                                                                                                             \
    }                                                                                                                 \
    _Pragma("unroll") for (int n = 0; n < NVC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        if (i < 32 * (DV / 8)) {                                                                                      \
            const int kk = i % 32, c = i / 32;                                                                        \
            const uint4 raw = rows[RB][kk] >= 0 ? vreg[n] : uint4{0u, 0u, 0u, 0u};                                    \
            const int k16 = kk & 15, rem = k16 & 7;                                                                   \
            const int place = (kk & 16) + 8 * (rem >> 2) + 4 * (k16 >> 3) + (rem & 3);                                \
            const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};                                                      \
            _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                           \
                Vt[(8 * c + 2 * e) * MT_VS + place] = (uint16_t)(wv[e] & 0xffffu);                                    \
                Vt[(8 * c + 2 * e + 1) * MT_VS + place] = (uint16_t)(wv[e] >> 16);                                    \
            }                                                                                                         \
        }                                                                                                             \
    }
    const int nblk_all = (n_keys + 31) / 32;
    const int b_begin = (int)((long)nblk_all * sp / nsplit), nblk = (int)((long)nblk_all * (sp + 1) / nsplit) - b_begin;
    if (threadIdx.x < 32) {
        rows[0][threadIdx.x] = row_of(32 * b_begin);
        rows[1][threadIdx.x] = row_of(32 * b_begin + 32);
        rows[2][threadIdx.x] = row_of(32 * b_begin + 64);
    }
    __syncthreads();
    MT_LOAD(0, kregA, vregA)
    MT_LOAD(1, kregB, vregB)
    MT_STORE(0, kregA, vregA)
    __syncthreads();
    // Block b is in LDS and block b + 1 in registers; block b + 2 is asked for before b is worked on, and the rows of
    // b + 3 before that: a trip to memory has two turns' time.  Two turns a trip, so that the registers of a turn are
    // a constant of the code.
    for (int b2 = 0; b2 < nblk; b2 += 2) {
#pragma unroll
      for (int turn = 0; turn < 2; ++turn) {
        const int b = b2 + turn;
        if (b >= nblk) break;
        const int i0 = 32 * (b_begin + b), rb = b & 3, rb1 = (b + 1) & 3, rb2 = (b + 2) & 3, rb3 = (b + 3) & 3;
        int ro3 = -1;
        if (threadIdx.x < 32) ro3 = row_of(i0 + 96);
        if (turn == 0) { MT_LOAD(rb2, kregA, vregA) } else { MT_LOAD(rb2, kregB, vregB) }     // (past the last block: rows -1, row 0 is read and never stored)
        if (active) {
            // ---- S^T = K Q^T
            ma_f32x16 sv;
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = 0.f;
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                ma_frag8 kf;
                kf.raw = *reinterpret_cast<const uint4*>(&Ks[ql * KROW + 16 * st + 8 * h]);
                sv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf.v, qf[st].v, sv, 0, 0, 0);
            }
            // ---- scale, cap, mask.  A block that every query of the tile sees whole (most are) needs no masks: its
            // places all have rows, it lies wholly among the kept positions or wholly inside every query's window.
            const bool whole = i0 + 31 < n_keys && !(i0 < n_first && i0 + 31 >= n_first) && __all(rows[rb][ql] >= 0) &&
                               (i0 + 31 < n_first || (visible_key(i0 + 31, n_first, lo_min) <= p0 && visible_key(i0, n_first, lo_min) >= lq_last));
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float sc = sv[r] * scale;
                if (softcap > 0.f) sc = softcap * fast_tanh(sc * inv_cap);
                sv[r] = sc;
            }
            if (!whole) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int place = 8 * (r >> 2) + 4 * h + (r & 3), i = i0 + place;
                    const int key = visible_key(i, n_first, lo_min);
                    const bool see = i < n_keys && rows[rb][place] >= 0 && key <= pq && (key >= lq || key < keep_first);
                    sv[r] = see ? sv[r] : -INFINITY;
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sv[r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, LI_WAVE));
            const float mn = fmaxf(m, mx);
            const float ms = (mn == -INFINITY) ? 0.f : mn;                    // a query may see no key of this block
            const float alpha = (m == -INFINITY) ? 1.f : fast_exp(m - ms);    // (m = -inf: nothing summed yet)
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) { sv[r] = fast_exp(sv[r] - ms); psum += sv[r]; }
            l = l * alpha + psum;
            m = mn;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
            }
            ma_frag8 pf[2];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) pf[st].w[i] = pack2_bf16(sv[8 * st + 2 * i], sv[8 * st + 2 * i + 1]);
            // ---- O^T += V^T P^T
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    ma_frag8 vf;
                    vf.raw = *reinterpret_cast<const uint4*>(&Vt[(32 * dt + ql) * MT_VS + 16 * st + 8 * h]);
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[st].v, acc[dt], 0, 0, 0);
                }
        }
        __syncthreads();                                                  // block b has been read
        if (b + 1 < nblk) {
            if (turn == 0) { MT_STORE(rb1, kregB, vregB) } else { MT_STORE(rb1, kregA, vregA) }
        }
        if (threadIdx.x < 32) rows[rb3][threadIdx.x] = ro3;
        __syncthreads();
      }
    }
#undef MT_LOAD
#undef MT_STORE
    if (!active) return;
    l += __shfl_xor(l, 32, LI_WAVE);
    if (ql >= ntok) return;
    if (nsplit > 1) {                              // this split's sums, maximum and sum of weights, for the join kernel
        float* part = parts + (((size_t)(t0 + ql) * nh + head) * nsplit + sp) * (DV + 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg)
            {                                      // (a part starts on 8 bytes)
                float2* dst = reinterpret_cast<float2*>(part + 32 * dt + 8 * rg + 4 * h);
                dst[0] = float2{acc[dt][4 * rg], acc[dt][4 * rg + 1]};
                dst[1] = float2{acc[dt][4 * rg + 2], acc[dt][4 * rg + 3]};
            }
        if (h == 0) { part[DV] = m; part[DV + 1] = l; }
        return;
    }
    const float inv = finish_factor(l, m, sink, gate, gate_stride, t0 + ql, head);
    bf16_t* orow = out + ((size_t)(t0 + ql) * nh + head) * DV;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {           // registers 4 rg .. 4 rg + 3: value columns 32 dt + 8 rg + 4 h ..
            uint32_t* dst = reinterpret_cast<uint32_t*>(orow + 32 * dt + 8 * rg + 4 * h);
            dst[0] = pack2_bf16(acc[dt][4 * rg] * inv, acc[dt][4 * rg + 1] * inv);
            dst[1] = pack2_bf16(acc[dt][4 * rg + 2] * inv, acc[dt][4 * rg + 3] * inv);
        }
}

__global__ void masked_attention_join_kernel(const float* __restrict__ parts, bf16_t* __restrict__ out,
                                             const int* __restrict__ token_list, int nh, int dv, int nsplit, const float* __restrict__ sink,
                                             const float* __restrict__ gate, long gate_stride, int by_token = 0);

// ------------------------------------------------------------------------------------------- single tokens, MFMA
// Decoding where a kv head serves many query heads (a compressed cache serves ALL of them): the same transposed
// tiles with the group's HEADS as the 32 columns, one wave a (token, kv head, 32 heads, split of the keys).  Every
// key of the token's list is visible to it, so only places past the split's end are masked.  The splits are
// joined by `masked_attention_join_kernel`.
template <int KS, int DT>
__global__ __launch_bounds__(64) void masked_attention_heads_kernel(
    const float* __restrict__ q, int q_token_stride, int q_head_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc, int k_row, int v_row,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_list,
    const int* __restrict__ seg_of_token, const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    int nh, int nkv, int page_size, int num_pages, int window, int keep_first, float softcap, float scale, const float* __restrict__ sink, const float* __restrict__ gate, long gate_stride,
    int nsplit, float* __restrict__ parts) {
    constexpr int DK = KS * 16, DV = DT * 32, KROW = DK + 8;
    constexpr int NT = 64;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[32 * KROW];       // [key place][dimension]
    __shared__ __attribute__((aligned(16))) uint16_t Vt[DV * MT_VS];      // [value column][key place, permuted]
    __shared__ int rows[3][32];                                           // the cache row of each key place of three blocks in turn, -1: none
    const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, kvh = blockIdx.y;
    const int s = seg_of_token[t];
    const int p0 = ctx_len[s] - q_len[s] + (t - q_start[s]);              // the token's position
    const int p_last = p0;
    const int lo_min = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    const int n_first = keep_first < lo_min ? keep_first : lo_min;
    const int n_all = n_first + (p_last - lo_min + 1);
    const int hc = blockIdx.z / nsplit, sp = blockIdx.z % nsplit;         // the chunk of 32 heads and the split of the keys
    const int i_begin = (int)((long)n_all * sp / nsplit), n_keys = (int)((long)n_all * (sp + 1) / nsplit);
    const int* table = block_table + (size_t)s * max_blocks;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, ql = lane & 31, h = lane >> 5;
    const int rep = nh / nkv;
    const int hq = hc * 32 + ql;                                          // this lane's head within the group (a column of the tile)
    const bool has = hq < rep;
    const bool active = true;
    const int head = kvh * rep + (has ? hq : 0);
    (void)w;
    const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;

    ma_frag8 qf[KS];
    {
        const float* qrow = q + (size_t)t * q_token_stride + (size_t)head * q_head_stride;
#pragma unroll
        for (int st = 0; st < KS; ++st) {
            const float4 a = *reinterpret_cast<const float4*>(qrow + 16 * st + 8 * h);
            const float4 b = *reinterpret_cast<const float4*>(qrow + 16 * st + 8 * h + 4);
            qf[st].w[0] = pack2_bf16(a.x, a.y); qf[st].w[1] = pack2_bf16(a.z, a.w);
            qf[st].w[2] = pack2_bf16(b.x, b.y); qf[st].w[3] = pack2_bf16(b.z, b.w);
        }
    }
    ma_f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    // The cache row of key place tid of the block of keys that starts at list index i0 (threads 0..31).
    auto row_of = [&](int i0) -> int {
        const int i = i0 + (int)threadIdx.x;
        if (i >= n_keys) return -1;
        const int key = visible_key(i, n_first, lo_min);
        const int page = table[key / page_size];
        return (page >= 0 && page < num_pages) ? (page * nkv + kvh) * page_size + key % page_size : -1;
    };
    constexpr int NKC = (32 * (DK / 8) + NT - 1) / NT, NVC = (32 * (DV / 8) + NT - 1) / NT;
    uint4 kreg[NKC], vreg[NVC];
    // a block's keys and values on their way: from memory into registers (a place without a row reads row 0 and
    // is zeroed when it is stored) ...
#define MT_LOAD(RB)                                                                                                   \
    _Pragma("unroll") for (int n = 0; n < NKC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        const int kk = (i / (DK / 8)) & 31, c = i % (DK / 8), ro = rows[RB][kk];                                      \
        kreg[n] = *reinterpret_cast<const uint4*>(kc + (size_t)(ro >= 0 ? ro : 0) * k_row + 8 * c);                   \
    }                                                                                                                 \
    _Pragma("unroll") for (int n = 0; n < NVC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        const int kk = i % 32, c = (i / 32) % (DV / 8), ro = rows[RB][kk];                                            \
        vreg[n] = *reinterpret_cast<const uint4*>(vc + (size_t)(ro >= 0 ? ro : 0) * v_row + 8 * c);                   \
    }
    // ... and from the registers into LDS: keys as they are, values transposed and in the operand's key order
#define MT_STORE(RB)                                                                                                  \
    _Pragma("unroll") for (int n = 0; n < NKC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        if (i < 32 * (DK / 8)) {                                                                                      \
            const int kk = i / (DK / 8), c = i % (DK / 8);                                                            \
            *reinterpret_cast<uint4*>(&Ks[kk * KROW + 8 * c]) = rows[RB][kk] >= 0 ? kreg[n] : uint4{0u, 0u, 0u, 0u};  \
        }                                                                                                             \
    }                                                                                                                 \
    _Pragma("unroll") for (int n = 0; n < NVC; ++n) {                                                                 \
        const int i = threadIdx.x + NT * n;                                                                           \
        if (i < 32 * (DV / 8)) {                                                                                      \
            const int kk = i % 32, c = i / 32;                                                                        \
            const uint4 raw = rows[RB][kk] >= 0 ? vreg[n] : uint4{0u, 0u, 0u, 0u};                                    \
            const int k16 = kk & 15, rem = k16 & 7;                                                                   \
            const int place = (kk & 16) + 8 * (rem >> 2) + 4 * (k16 >> 3) + (rem & 3);                                \
            const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};                                                      \
            _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                           \
                Vt[(8 * c + 2 * e) * MT_VS + place] = (uint16_t)(wv[e] & 0xffffu);                                    \
                Vt[(8 * c + 2 * e + 1) * MT_VS + place] = (uint16_t)(wv[e] >> 16);                                    \
            }                                                                                                         \
        }                                                                                                             \
    }
    const int nblk = (n_keys - i_begin + 31) / 32;
    if (threadIdx.x < 32) {
        rows[0][threadIdx.x] = row_of(i_begin);
        rows[1][threadIdx.x] = row_of(i_begin + 32);
    }
    __syncthreads();
    MT_LOAD(0)
    MT_STORE(0)
    __syncthreads();
    // block b is in LDS; block b + 1 is asked for before b is worked on, and the rows of b + 2 before that
    for (int b = 0; b < nblk; ++b) {
        const int i0 = i_begin + 32 * b, rb = b % 3, rb1 = (b + 1) % 3, rb2 = (b + 2) % 3;
        int ro2 = -1;
        if (threadIdx.x < 32) ro2 = row_of(i0 + 64);
        MT_LOAD(rb1)                                                      // (past the last block: its rows are -1, row 0 is read and never stored)
        if (active) {
            // ---- S^T = K Q^T
            ma_f32x16 sv;
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = 0.f;
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                ma_frag8 kf;
                kf.raw = *reinterpret_cast<const uint4*>(&Ks[ql * KROW + 16 * st + 8 * h]);
                sv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf.v, qf[st].v, sv, 0, 0, 0);
            }
            // ---- scale, cap, mask.  A block that every query of the tile sees whole (most are) needs no masks: its
            // places all have rows, it lies wholly among the kept positions or wholly inside every query's window.
            const bool whole = i0 + 31 < n_keys && __all(rows[rb][ql] >= 0);      // (every listed key is visible to the token)
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float sc = sv[r] * scale;
                if (softcap > 0.f) sc = softcap * fast_tanh(sc * inv_cap);
                sv[r] = sc;
            }
            if (!whole) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int place = 8 * (r >> 2) + 4 * h + (r & 3), i = i0 + place;
                    const bool see = i < n_keys && rows[rb][place] >= 0;
                    sv[r] = see ? sv[r] : -INFINITY;
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sv[r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, LI_WAVE));
            const float mn = fmaxf(m, mx);
            const float ms = (mn == -INFINITY) ? 0.f : mn;                    // a query may see no key of this block
            const float alpha = (m == -INFINITY) ? 1.f : fast_exp(m - ms);    // (m = -inf: nothing summed yet)
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) { sv[r] = fast_exp(sv[r] - ms); psum += sv[r]; }
            l = l * alpha + psum;
            m = mn;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
            }
            ma_frag8 pf[2];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) pf[st].w[i] = pack2_bf16(sv[8 * st + 2 * i], sv[8 * st + 2 * i + 1]);
            // ---- O^T += V^T P^T
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    ma_frag8 vf;
                    vf.raw = *reinterpret_cast<const uint4*>(&Vt[(32 * dt + ql) * MT_VS + 16 * st + 8 * h]);
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[st].v, acc[dt], 0, 0, 0);
                }
        }
        __syncthreads();                                                  // block b has been read
        if (b + 1 < nblk) { MT_STORE(rb1) }
        if (threadIdx.x < 32) rows[rb2][threadIdx.x] = ro2;
        __syncthreads();
    }
#undef MT_LOAD
#undef MT_STORE
    l += __shfl_xor(l, 32, LI_WAVE);
    if (!has) return;
    if (nsplit == 1) {
        const float inv = finish_factor(l, m, sink, gate, gate_stride, t, head);
        bf16_t* orow = out + ((size_t)t * nh + head) * DV;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {       // registers 4 rg .. 4 rg + 3: value columns 32 dt + 8 rg + 4 h ..
                uint32_t* dst = reinterpret_cast<uint32_t*>(orow + 32 * dt + 8 * rg + 4 * h);
                dst[0] = pack2_bf16(acc[dt][4 * rg] * inv, acc[dt][4 * rg + 1] * inv);
                dst[1] = pack2_bf16(acc[dt][4 * rg + 2] * inv, acc[dt][4 * rg + 3] * inv);
            }
    } else {                                       // this split's sums, maximum and sum of weights, for the join kernel
        float* part = parts + (((size_t)blockIdx.x * nh + head) * nsplit + sp) * (DV + 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg)
#pragma unroll
                for (int e = 0; e < 4; ++e) part[32 * dt + 8 * rg + 4 * h + e] = acc[dt][4 * rg + e];
        if (h == 0) { part[DV] = m; part[DV + 1] = l; }
    }
}

// 1 if the tile kernel takes these sizes (bfloat16 cache and output)
extern "C" int li_masked_attention_tiles_takes(int dk, int dv) {
#define MT_HAS(K, V) if (dk == K && dv == V) return 1;
    MT_HAS(64, 64) MT_HAS(128, 128) MT_HAS(128, 64) MT_HAS(64, 128) MT_HAS(96, 64) MT_HAS(160, 128) MT_HAS(192, 128)
    MT_HAS(256, 256) MT_HAS(320, 256) MT_HAS(288, 256)
#undef MT_HAS
    return 0;
}

extern "C" int li_masked_attention_tiles(const float* q, int q_token_stride, int q_head_stride, void* out, const void* kc,
                                         const void* vc, int k_row, int v_row, const int* block_table, int max_blocks,
                                         const int* tiles, int num_tiles, const int* q_start, const int* q_len,
                                         const int* ctx_len, int nh, int nkv, int dk, int dv, int page_size, int num_pages,
                                         int window, int keep_first, float softcap, float scale, const float* sink, const float* gate, long gate_stride, int nsplit, float* parts,
                                         long parts_floats, const int* multi_tokens, int num_multi, int num_tokens,
                                         hipStream_t stream) {
    if (num_tiles <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || nkv > 65535 || dk > k_row || dv > v_row || page_size <= 0 ||
        window < 0 || keep_first < 0 || max_blocks <= 0 || k_row % 8 || v_row % 8 || q_token_stride % 4 || q_head_stride % 4 ||
        ((uintptr_t)q | (uintptr_t)kc | (uintptr_t)vc) % 16 || (uintptr_t)out % 8 || !li_masked_attention_tiles_takes(dk, dv) ||
        nsplit < 1 || nsplit > 16 || num_multi <= 0 ||
        (nsplit > 1 && (!parts || (uintptr_t)parts % 8 || parts_floats < (long)num_tokens * nh * nsplit * (dv + 2))))
        return LI_ERR_SIZE;
    const int rep = nh / nkv;
    // five to eight heads a kv head: one block of eight waves (one staging of every block of keys for all of them)
    // rather than blocks of four and of one to four; more heads: whichever leaves fewer waves idle
    const int nw = (rep > 4 && (rep <= 8 || rep % 8 == 0 || rep % 8 > 4)) ? 8 : 4;
    const dim3 grid(num_tiles, nkv, ((rep + nw - 1) / nw) * nsplit);
#define MT_GO(K, V)                                                                                                        \
    if (dk == K && dv == V) {                                                                                              \
        if (nw == 8)                                                                                                       \
            masked_attention_tile_kernel<K / 16, V / 32, 8><<<grid, 512, 0, stream>>>(                                     \
                q, q_token_stride, q_head_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, k_row, v_row, block_table, \
                max_blocks, tiles, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, keep_first, softcap, scale, sink, gate, gate_stride, \
                nsplit, parts);                                                                                            \
        else                                                                                                               \
            masked_attention_tile_kernel<K / 16, V / 32, 4><<<grid, 256, 0, stream>>>(                                     \
                q, q_token_stride, q_head_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, k_row, v_row, block_table, \
                max_blocks, tiles, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, keep_first, softcap, scale, sink, gate, gate_stride, \
                nsplit, parts);                                                                                            \
        if (nsplit > 1)                                                                                                    \
            masked_attention_join_kernel<<<dim3(num_multi, nh), dv >= 256 ? 256 : 128, 0, stream>>>(parts, (bf16_t*)out, multi_tokens, nh, dv, nsplit, sink, gate, gate_stride, 1); \
        return li_launch_status();                                                                                         \
    }
    MT_GO(64, 64) MT_GO(128, 128) MT_GO(128, 64) MT_GO(64, 128) MT_GO(96, 64) MT_GO(160, 128) MT_GO(192, 128)
    MT_GO(256, 256) MT_GO(320, 256) MT_GO(288, 256)
#undef MT_GO
    return LI_ERR_SIZE;
}


extern "C" int li_masked_attention_heads(const float* q, int q_token_stride, int q_head_stride, void* out, const void* kc,
                                         const void* vc, int k_row, int v_row, const int* block_table, int max_blocks,
                                         const int* token_list, int n_tokens, const int* seg_of_token, const int* q_start,
                                         const int* q_len, const int* ctx_len, int nh, int nkv, int dk, int dv, int page_size,
                                         int num_pages, int window, int keep_first, float softcap, float scale, const float* sink, const float* gate, long gate_stride, int nsplit,
                                         float* parts, long parts_floats, hipStream_t stream) {
    if (n_tokens <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || nkv > 65535 || dk > k_row || dv > v_row || page_size <= 0 ||
        window < 0 || keep_first < 0 || max_blocks <= 0 || k_row % 8 || v_row % 8 || q_token_stride % 4 || q_head_stride % 4 ||
        ((uintptr_t)q | (uintptr_t)kc | (uintptr_t)vc) % 16 || (uintptr_t)out % 8 || !li_masked_attention_tiles_takes(dk, dv) ||
        nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!parts || parts_floats < (long)n_tokens * nh * nsplit * (dv + 2))))
        return LI_ERR_SIZE;
    const int rep = nh / nkv;
    const dim3 grid(n_tokens, nkv, ((rep + 31) / 32) * nsplit);
#define MH_GO(K, V)                                                                                                        \
    if (dk == K && dv == V) {                                                                                              \
        masked_attention_heads_kernel<K / 16, V / 32><<<grid, 64, 0, stream>>>(                                            \
            q, q_token_stride, q_head_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, k_row, v_row, block_table, \
            max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, keep_first, \
            softcap, scale, sink, gate, gate_stride, nsplit, parts);                                                                                \
        if (nsplit > 1)                                                                                                    \
            masked_attention_join_kernel<<<dim3(n_tokens, nh), dv >= 256 ? 256 : 128, 0, stream>>>(parts, (bf16_t*)out, token_list, nh, dv, nsplit, sink, gate, gate_stride); \
        return li_launch_status();                                                                                         \
    }
    MH_GO(64, 64) MH_GO(128, 128) MH_GO(128, 64) MH_GO(64, 128) MH_GO(96, 64) MH_GO(160, 128) MH_GO(192, 128)
    MH_GO(256, 256) MH_GO(320, 256) MH_GO(288, 256)
#undef MH_GO
    return LI_ERR_SIZE;
}

// ------------------------------------------------------------------------------------------- single tokens, bfloat16
// Decoding: one query a request, so the work is reading its visible keys and values once.  A block of four waves
// takes one (token, kv head) and RH query heads of that kv head, so that a row is read once for all of them.  A
// key's row is spread over 8 lanes, 16 bytes a lane and piece (lane j holds the pieces j, j + 8, ...): a wave takes
// 8 keys at a time, the block 32, and U such rounds are in flight.  Every group of 8 lanes keeps a running
// (maximum, sum, sums of values) per head over its keys; the groups of a wave are joined by a butterfly, the waves
// through LDS in wave order.
// the sum over a group of 8 neighbouring lanes, in every lane of the group, by lane moves inside the vector ALU
// (quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror) instead of three trips through LDS
__device__ __forceinline__ float dpp_move(float v, const int ctrl) {
    if (ctrl == 0xB1) return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
    if (ctrl == 0x4E) return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
}
__device__ __forceinline__ float sum_over_8_lanes(float d) {
    d += dpp_move(d, 0xB1);
    d += dpp_move(d, 0x4E);
    d += dpp_move(d, 0x141);
    return d;
}

__device__ __forceinline__ void unpack8(const uint4 raw, float* f) {
    f[0] = __uint_as_float(raw.x << 16); f[1] = __uint_as_float(raw.x & 0xffff0000u);
    f[2] = __uint_as_float(raw.y << 16); f[3] = __uint_as_float(raw.y & 0xffff0000u);
    f[4] = __uint_as_float(raw.z << 16); f[5] = __uint_as_float(raw.z & 0xffff0000u);
    f[6] = __uint_as_float(raw.w << 16); f[7] = __uint_as_float(raw.w & 0xffff0000u);
}

template <int NPK, int NPV, int RH, int U>
__global__ __launch_bounds__(256) void masked_attention_single_kernel(
    const float* __restrict__ q, int q_token_stride, int q_head_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc, int k_row, int v_row,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_list,
    const int* __restrict__ seg_of_token, const int* __restrict__ q_start, const int* __restrict__ q_len,
    const int* __restrict__ ctx_len, int nh, int nkv, int dk, int dv, int page_size, int num_pages, int window,
    int keep_first, float softcap, float scale, const float* __restrict__ sink, const float* __restrict__ gate, long gate_stride, int tab_cap, int pshift, int nsplit, float* __restrict__ parts) {
    extern __shared__ float join[];                 // [4 waves][RH][dv + 2], then tab_cap table entries
    int* tab = (int*)(join + (size_t)4 * RH * (dv + 2));
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, g = lane >> 3, j = lane & 7;
    const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, kvh = blockIdx.y;
    const int rep = nh / nkv, hfirst = (blockIdx.z / nsplit) * RH, sp = blockIdx.z % nsplit;
    const int nheads = rep - hfirst < RH ? rep - hfirst : RH;
    const int s = seg_of_token[t];
    const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_first = keep_first < lo ? keep_first : lo;
    const int n_all = n_first + (p - lo + 1);
    // this block's share of the visible keys (split sp of nsplit)
    const int i_begin = (int)((long)n_all * sp / nsplit), n_keys = (int)((long)n_all * (sp + 1) / nsplit);
    const int* table = block_table + (size_t)s * max_blocks;
    // the pages of the visible keys in LDS (the window's blocks, then the kept first blocks), so that a key's row
    // costs no trip to memory before its own; a table too long for the room given is read where it lies
    const int b_lo = pshift >= 0 ? lo >> pshift : lo / page_size, b_hi = pshift >= 0 ? p >> pshift : p / page_size;
    const int nb_w = b_hi - b_lo + 1, nb_k = n_first > 0 ? (n_first - 1) / page_size + 1 : 0;
    const bool in_lds = nb_w + nb_k <= tab_cap;
    if (in_lds) {
        for (int i = threadIdx.x; i < nb_w; i += 256) tab[i] = table[b_lo + i];
        for (int i = threadIdx.x; i < nb_k; i += 256) tab[nb_w + i] = table[i];
    }
    __syncthreads();

    float qr[RH][NPK][8];
#pragma unroll
    for (int hh = 0; hh < RH; ++hh) {
        const float* qrow = q + (size_t)t * q_token_stride + (size_t)(kvh * rep + hfirst + (hh < nheads ? hh : 0)) * q_head_stride;
#pragma unroll
        for (int c = 0; c < NPK; ++c) {
            const int d0 = 8 * (j + 8 * c);
            const bool on = d0 < dk && hh < nheads;
            const float4 a = on ? *reinterpret_cast<const float4*>(qrow + d0) : float4{0.f, 0.f, 0.f, 0.f};
            const float4 b = on ? *reinterpret_cast<const float4*>(qrow + d0 + 4) : float4{0.f, 0.f, 0.f, 0.f};
            qr[hh][c][0] = a.x; qr[hh][c][1] = a.y; qr[hh][c][2] = a.z; qr[hh][c][3] = a.w;
            qr[hh][c][4] = b.x; qr[hh][c][5] = b.y; qr[hh][c][6] = b.z; qr[hh][c][7] = b.w;
        }
    }
    float acc[RH][NPV][8];
    float m[RH], l[RH];
#pragma unroll
    for (int hh = 0; hh < RH; ++hh) {
        m[hh] = -INFINITY; l[hh] = 0.f;
#pragma unroll
        for (int c = 0; c < NPV; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[hh][c][e] = 0.f;
    }
    const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
    // the rows of a round's keys (a key past the last: row 0, read and not used) and their pieces; the next round's
    // are asked for before this round's are used, without a condition (a load under a condition would make every
    // later use wait for all loads)
    size_t ro[U];
    bool ok[U];
    uint4 kp[U][NPK], vp[U][NPV];
#define MS_ROWS(I0, RO, OK)                                                                                          \
    _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                                  \
        const int i = (I0) + 32 * u + 8 * w + g;                                                                     \
        OK[u] = i < n_keys;                                                                                          \
        const int ii = OK[u] ? i : 0;                                                                                \
        const int key = visible_key(ii, n_first, lo);                                                                \
        const int blk = pshift >= 0 ? key >> pshift : key / page_size;                                               \
        const int page = in_lds ? tab[ii < n_first ? nb_w + blk : blk - b_lo] : table[blk];                          \
        OK[u] = OK[u] && page >= 0 && page < num_pages;                                                              \
        RO[u] = OK[u] ? (size_t)(page * nkv + kvh) * page_size + (key - blk * page_size) : 0;                        \
    }
#define MS_FETCH(RO, KP, VP)                                                                                         \
    _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                                  \
        _Pragma("unroll") for (int c = 0; c < NPK; ++c) {                                                            \
            const int d0 = 8 * (j + 8 * c);                                                                          \
            KP[u][c] = *reinterpret_cast<const uint4*>(kc + RO[u] * k_row + (d0 < dk ? d0 : 0));                     \
        }                                                                                                            \
        _Pragma("unroll") for (int c = 0; c < NPV; ++c) {                                                            \
            const int d0 = 8 * (j + 8 * c);                                                                          \
            VP[u][c] = *reinterpret_cast<const uint4*>(vc + RO[u] * v_row + (d0 < dv ? d0 : 0));                     \
        }                                                                                                            \
    }
    MS_ROWS(i_begin, ro, ok)
    MS_FETCH(ro, kp, vp)
    for (int i0 = i_begin; i0 < n_keys; i0 += 32 * U) {
        size_t ro2[U];
        bool ok2[U];
        uint4 kp2[U][NPK], vp2[U][NPV];
        MS_ROWS(i0 + 32 * U, ro2, ok2)
        MS_FETCH(ro2, kp2, vp2)
        float sc[U][RH];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[NPK][8];
#pragma unroll
            for (int c = 0; c < NPK; ++c) unpack8(kp[u][c], kf[c]);
#pragma unroll
            for (int hh = 0; hh < RH; ++hh) {
                float d = 0.f;
#pragma unroll
                for (int c = 0; c < NPK; ++c)
#pragma unroll
                    for (int e = 0; e < 8; ++e) d = fmaf(qr[hh][c][e], kf[c][e], d);      // (pieces past dk meet zeros of q)
                d = sum_over_8_lanes(d) * scale;
                if (softcap > 0.f) d = softcap * fast_tanh(d * inv_cap);
                sc[u][hh] = ok[u] ? d : -INFINITY;
            }
        }
#pragma unroll
        for (int hh = 0; hh < RH; ++hh) {
            float mx = sc[0][hh];
#pragma unroll
            for (int u = 1; u < U; ++u) mx = fmaxf(mx, sc[u][hh]);
            const float mn = fmaxf(m[hh], mx);
            const float ms = (mn == -INFINITY) ? 0.f : mn;
            const float alpha = (m[hh] == -INFINITY) ? 0.f : fast_exp(m[hh] - ms);
            float pu[U], psum = 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) { pu[u] = fast_exp(sc[u][hh] - ms); psum += pu[u]; }
            l[hh] = l[hh] * alpha + psum;
            m[hh] = mn;
#pragma unroll
            for (int c = 0; c < NPV; ++c) {
                float a8[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) a8[e] = acc[hh][c][e] * alpha;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    float vf[8];
                    unpack8(vp[u][c], vf);
#pragma unroll
                    for (int e = 0; e < 8; ++e) a8[e] = fmaf(pu[u], vf[e], a8[e]);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[hh][c][e] = a8[e];
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            ok[u] = ok2[u];
#pragma unroll
            for (int c = 0; c < NPK; ++c) kp[u][c] = kp2[u][c];
#pragma unroll
            for (int c = 0; c < NPV; ++c) vp[u][c] = vp2[u][c];
        }
    }
#undef MS_ROWS
#undef MS_FETCH
    // the groups of a wave
#pragma unroll
    for (int off = 8; off < 64; off <<= 1) {
#pragma unroll
        for (int hh = 0; hh < RH; ++hh) {
            const float m2 = __shfl_xor(m[hh], off, LI_WAVE), l2 = __shfl_xor(l[hh], off, LI_WAVE);
            const float mn = fmaxf(m[hh], m2);
            const float f1 = (m[hh] == -INFINITY) ? 0.f : expf(m[hh] - mn), f2 = (m2 == -INFINITY) ? 0.f : expf(m2 - mn);
            l[hh] = l[hh] * f1 + l2 * f2;
            m[hh] = mn;
#pragma unroll
            for (int c = 0; c < NPV; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[hh][c][e] = acc[hh][c][e] * f1 + __shfl_xor(acc[hh][c][e], off, LI_WAVE) * f2;
        }
    }
    // the waves
    if (g == 0) {
#pragma unroll
        for (int hh = 0; hh < RH; ++hh) {
            float* mine = join + (size_t)(w * RH + hh) * (dv + 2);
            if (j == 0) { mine[dv] = m[hh]; mine[dv + 1] = l[hh]; }
#pragma unroll
            for (int c = 0; c < NPV; ++c) {
                const int d0 = 8 * (j + 8 * c);
                if (d0 < dv)
#pragma unroll
                    for (int e = 0; e < 8; ++e) mine[d0 + e] = acc[hh][c][e];
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nheads * dv; idx += 256) {
        const int hh = idx / dv, d = idx % dv;
        float mm = -INFINITY;
#pragma unroll
        for (int x = 0; x < 4; ++x) mm = fmaxf(mm, join[(size_t)(x * RH + hh) * (dv + 2) + dv]);
        float a = 0.f, ll = 0.f;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const float* r = join + (size_t)(x * RH + hh) * (dv + 2);
            const float f = (r[dv] == -INFINITY) ? 0.f : expf(r[dv] - mm);
            a += r[d] * f;
            ll += r[dv + 1] * f;
        }
        const int head = kvh * rep + hfirst + hh;
        if (nsplit == 1) {
            out[((size_t)t * nh + head) * dv + d].bits = float_to_bf16(a * finish_factor(ll, mm, sink, gate, gate_stride, t, head));
        } else {                                    // this split's sums, maximum and sum of weights: joined by the kernel behind
            float* part = parts + (((size_t)blockIdx.x * nh + head) * nsplit + sp) * (dv + 2);
            part[d] = a;
            if (d == 0) { part[dv] = mm; part[dv + 1] = ll; }
        }
    }
}

// joins the splits of every (token, head) in split order: a block a (token, head)
// (the parts of a token lie at its place in the list, or, with by_token, at its own number)
__global__ void masked_attention_join_kernel(const float* __restrict__ parts, bf16_t* __restrict__ out,
                                             const int* __restrict__ token_list, int nh, int dv, int nsplit, const float* __restrict__ sink,
                                             const float* __restrict__ gate, long gate_stride, int by_token) {
    const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, head = blockIdx.y;
    const float* base = parts + ((size_t)(by_token ? t : (int)blockIdx.x) * nh + head) * nsplit * (dv + 2);
    float mm = -INFINITY;
    for (int x = 0; x < nsplit; ++x) mm = fmaxf(mm, base[(size_t)x * (dv + 2) + dv]);
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        float a = 0.f, ll = 0.f;
        for (int x = 0; x < nsplit; ++x) {
            const float* r = base + (size_t)x * (dv + 2);
            const float f = (r[dv] == -INFINITY) ? 0.f : expf(r[dv] - mm);
            a += r[d] * f;
            ll += r[dv + 1] * f;
        }
        out[((size_t)t * nh + head) * dv + d].bits = float_to_bf16(a * finish_factor(ll, mm, sink, gate, gate_stride, t, head));
    }
}

// 1 if the kernel for single tokens takes these sizes (bfloat16 cache and output)
extern "C" int li_masked_attention_single_takes(int dk, int dv) {
    const int npk = (dk + 63) / 64, npv = (dv + 63) / 64;
    if (dk % 8 || dv % 8 || dk <= 0 || dv <= 0) return 0;
    return (npk <= 2 && npv <= 2) || (npk == 3 && npv == 2) || (npk == 4 && npv == 4) || (npk == 5 && npv == 4) || (npk == 4 && npv == 3);
}

// blocks that a call launches per split (the host sizes the number of splits by it)
extern "C" int li_masked_attention_single_blocks(int n_tokens, int nh, int nkv, int dk, int dv) {
    const int rep = nh / nkv, npk = (dk + 63) / 64, npv = (dv + 63) / 64;
    const int rh = (npk + npv > 6) ? (rep >= 2 ? 2 : 1) : (rep >= 4 && (rep % 4 == 0 || rep % 4 == 3 || rep > 8)) ? 4 : rep >= 2 ? 2 : 1;
    return n_tokens * nkv * ((rep + rh - 1) / rh);
}

extern "C" int li_masked_attention_single(const float* q, int q_token_stride, int q_head_stride, void* out, const void* kc,
                                          const void* vc, int k_row, int v_row, const int* block_table, int max_blocks,
                                          const int* token_list, int n_tokens, const int* seg_of_token, const int* q_start,
                                          const int* q_len, const int* ctx_len, int nh, int nkv, int dk, int dv, int page_size,
                                          int num_pages, int window, int keep_first, float softcap, float scale, const float* sink, const float* gate, long gate_stride,
                                          int nsplit, float* parts, long parts_floats, hipStream_t stream) {
    if (n_tokens <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || nkv > 65535 || dk > k_row || dv > v_row || page_size <= 0 ||
        window < 0 || keep_first < 0 || max_blocks <= 0 || num_pages <= 0 || k_row % 8 || v_row % 8 || q_token_stride % 4 ||
        q_head_stride % 4 || ((uintptr_t)q | (uintptr_t)kc | (uintptr_t)vc) % 16 || !li_masked_attention_single_takes(dk, dv))
        return LI_ERR_SIZE;
    const int rep = nh / nkv, npk = (dk + 63) / 64, npv = (dv + 63) / 64;
    const int rh = (npk + npv > 6) ? (rep >= 2 ? 2 : 1) : (rep >= 4 && (rep % 4 == 0 || rep % 4 == 3 || rep > 8)) ? 4 : rep >= 2 ? 2 : 1;
    if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!parts || parts_floats < (long)n_tokens * nh * nsplit * (dv + 2)))) return LI_ERR_SIZE;
    const dim3 grid(n_tokens, nkv, ((rep + rh - 1) / rh) * nsplit);
    // room for the pages of one query's visible keys: the window's and the kept ones, or the whole table's width
    long cap = window > 0 ? (long)window / page_size + 3 + (keep_first + page_size - 1) / page_size : (long)max_blocks;
    if (cap > 12288) cap = 0;                       // (longer tables are read where they lie)
    const int tab_cap = (int)cap;
    int pshift = -1;
    for (int b = 0; b < 31; ++b) if (page_size == (1 << b)) pshift = b;
    const size_t lds = (size_t)4 * rh * (dv + 2) * 4 + (size_t)tab_cap * 4;
#define MS_GO(K, V, R, UU)                                                                                                  \
    masked_attention_single_kernel<K, V, R, UU><<<grid, 256, lds, stream>>>(                                                \
        q, q_token_stride, q_head_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, k_row, v_row, block_table,    \
        max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, nh, nkv, dk, dv, page_size, num_pages, window,       \
        keep_first, softcap, scale, sink, gate, gate_stride, tab_cap, pshift, nsplit, parts)
#define MS_JOIN                                                                                                             \
    if (nsplit > 1)                                                                                                         \
        masked_attention_join_kernel<<<dim3(n_tokens, nh), dv >= 256 ? 256 : 128, 0, stream>>>(parts, (bf16_t*)out, token_list, nh, dv, nsplit, sink, gate, gate_stride);
#define MS_SMALL(K, V)                                                                                                      \
    if (npk == K && npv == V) {                                                                                             \
        if (rh == 4) MS_GO(K, V, 4, 4); else if (rh == 2) MS_GO(K, V, 2, 4); else MS_GO(K, V, 1, 4);                        \
        MS_JOIN                                                                                                             \
        return li_launch_status();                                                                                          \
    }
#define MS_LARGE(K, V)                                                                                                      \
    if (npk == K && npv == V) {                                                                                             \
        if (rh == 2) MS_GO(K, V, 2, 2); else MS_GO(K, V, 1, 2);                                                             \
        MS_JOIN                                                                                                             \
        return li_launch_status();                                                                                          \
    }
    MS_SMALL(1, 1) MS_SMALL(2, 1) MS_SMALL(1, 2) MS_SMALL(2, 2) MS_SMALL(3, 2)
    MS_LARGE(4, 4) MS_LARGE(5, 4) MS_LARGE(4, 3)
#undef MS_GO
#undef MS_JOIN
#undef MS_SMALL
#undef MS_LARGE
    return LI_ERR_SIZE;
}

// ------------------------------------------------------------------------------------------- per-head products
// out[t, h, j] = sum_k m[h, j, k] * x[t, h, k]: every head has a matrix of its own, [n_out, n_in], stored one after
// the other.  x and out are addressed by a token stride and a head stride, so that a head's columns may lie inside
// a wider row.  With `gate`, head h's outputs of token t are multiplied by sigmoid(gate[t * gate_stride + h]).
// A block takes one head, HL_TOK tokens and 256 outputs: the tokens' inputs lie in LDS as float32, a
// thread owns an output and reads its matrix row once for all the tokens.  Sums are float32, in the order of k.
#define HL_TOK 8

// Behind a head's n_in inputs may lie `n` more columns that are not multiplied but ROTATED by the token's angles
// (cos, sin [T, n / 2]) and written behind the head's n_out outputs: pairs of neighbouring columns, or (split)
// column i with column i + n / 2.
struct HeadTail { int n; int split; const float* cosv; const float* sinv; };

template <typename TX, typename TO>
__device__ __forceinline__ void head_tail_rotate(const TX* __restrict__ src, TO* __restrict__ dst, int t, int i, const HeadTail& tail) {
    const int half = tail.n / 2, a = tail.split ? i : 2 * i, b = tail.split ? i + half : 2 * i + 1;
    const float c = tail.cosv[(size_t)t * half + i], sn = tail.sinv[(size_t)t * half + i];
    const float u = load_as_float(src + a), v = load_as_float(src + b);
    store_from_float(dst + a, fmaf(u, c, -__fmul_rn(v, sn)));
    store_from_float(dst + b, fmaf(v, c, __fmul_rn(u, sn)));
}

template <typename TX, typename TM, typename TO, bool VEC>
__global__ __launch_bounds__(256) void headwise_linear_kernel(
    const TX* __restrict__ x, long x_token_stride, int x_head_stride, const TM* __restrict__ m, TO* __restrict__ out,
    long o_token_stride, int o_head_stride, int T_, int n_out, int n_in, const float* __restrict__ gate, long gate_stride,
    HeadTail tail) {
    extern __shared__ float xs[];                    // [HL_TOK][n_in]
    const int h = blockIdx.y, t0 = blockIdx.x * HL_TOK;
    const int nt = (T_ - t0 < HL_TOK) ? T_ - t0 : HL_TOK;
    if (tail.n > 0 && blockIdx.z == 0)
        for (int u = threadIdx.x; u < nt * (tail.n / 2); u += 256) {
            const int tt = u / (tail.n / 2), i = u % (tail.n / 2);
            head_tail_rotate(x + (size_t)(t0 + tt) * x_token_stride + (size_t)h * x_head_stride + n_in,
                             out + (size_t)(t0 + tt) * o_token_stride + (size_t)h * o_head_stride + n_out, t0 + tt, i, tail);
        }
    for (int i = threadIdx.x; i < HL_TOK * n_in; i += 256) {
        const int tt = i / n_in, k = i % n_in;
        xs[i] = tt < nt ? load_as_float(x + (size_t)(t0 + tt) * x_token_stride + (size_t)h * x_head_stride + k) : 0.f;
    }
    // the heads' gates are asked for before the products, so that they have arrived when the outputs are ready
    float gf[HL_TOK];
#pragma unroll
    for (int tt = 0; tt < HL_TOK; ++tt) gf[tt] = gate ? gate[(size_t)(t0 + (tt < nt ? tt : 0)) * gate_stride + h] : 0.f;
    __syncthreads();
    // four neighbouring threads share an output: each takes every fourth piece of the matrix row
    constexpr int E = VEC ? 16 / (int)sizeof(TM) : 1;
    const int part = threadIdx.x & 3;
    for (int j = blockIdx.z * 64 + (threadIdx.x >> 2); j < n_out + 63; j += gridDim.z * 64) {       // (whole groups of four go round together)
        const bool on = j < n_out;
        const TM* row = m + ((size_t)h * n_out + (on ? j : 0)) * n_in;
        float acc[HL_TOK];
#pragma unroll
        for (int tt = 0; tt < HL_TOK; ++tt) acc[tt] = 0.f;
        for (int k = part * E; k < n_in; k += 4 * E) {
            float wv[E];
            if constexpr (VEC) {
                const uint4 raw = *reinterpret_cast<const uint4*>(row + k);
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
            } else {
                wv[0] = load_as_float(row + k);
            }
#pragma unroll
            for (int e = 0; e < E; ++e)
#pragma unroll
                for (int tt = 0; tt < HL_TOK; ++tt) acc[tt] = fmaf(wv[e], xs[tt * n_in + k + e], acc[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < HL_TOK; ++tt) {
            acc[tt] += __shfl_xor(acc[tt], 1, LI_WAVE);
            acc[tt] += __shfl_xor(acc[tt], 2, LI_WAVE);
        }
        if (on && part == 0)
            for (int tt = 0; tt < nt; ++tt) {
                const float f = gate ? 1.0f / (1.0f + expf(-gf[tt])) : 1.0f;
                store_from_float(out + (size_t)(t0 + tt) * o_token_stride + (size_t)h * o_head_stride + j, acc[tt] * f);
            }
    }
}

// The same product on the matrix cores, for bfloat16 matrices with n_in a multiple of 16 and n_out a multiple of
// 32: a wave takes 32 tokens and 32 outputs of one head and works on the transposed tile (outputs x tokens), so
// that both operands are 16-byte pieces of rows as they lie in memory (a matrix row's k-values; a token's
// inputs, rounded to bfloat16 if they are float32) and a lane ends with four consecutive outputs of its token.
template <typename TX, typename TO>
__global__ __launch_bounds__(256) void headwise_linear_mfma_kernel(
    const TX* __restrict__ x, long x_token_stride, int x_head_stride, const bf16_t* __restrict__ m, TO* __restrict__ out,
    long o_token_stride, int o_head_stride, int T_, int n_out, int n_in, const float* __restrict__ gate, long gate_stride,
    HeadTail tail) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, ql = lane & 31, h2 = lane >> 5;
    const int head = blockIdx.y, t0 = blockIdx.x * 32;
    if (tail.n > 0 && blockIdx.z == 0) {
        const int nt = (T_ - t0 < 32) ? T_ - t0 : 32;
        for (int u = threadIdx.x; u < nt * (tail.n / 2); u += 256) {
            const int tt = u / (tail.n / 2), i = u % (tail.n / 2);
            head_tail_rotate(x + (size_t)(t0 + tt) * x_token_stride + (size_t)head * x_head_stride + n_in,
                             out + (size_t)(t0 + tt) * o_token_stride + (size_t)head * o_head_stride + n_out, t0 + tt, i, tail);
        }
    }
    const int j0 = (blockIdx.z * 4 + w) * 32;
    if (j0 >= n_out) return;
    const int tok = t0 + ql < T_ ? t0 + ql : T_ - 1;
    const TX* xrow = x + (size_t)tok * x_token_stride + (size_t)head * x_head_stride + 8 * h2;
    const bf16_t* mrow = m + ((size_t)head * n_out + j0 + ql) * n_in + 8 * h2;
    ma_f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    for (int k = 0; k < n_in; k += 16) {
        ma_frag8 a, b;
        a.raw = *reinterpret_cast<const uint4*>(mrow + k);
        if constexpr (sizeof(TX) == 2) {
            b.raw = *reinterpret_cast<const uint4*>(xrow + k);
        } else {
            const float4 u = *reinterpret_cast<const float4*>(xrow + k);
            const float4 v = *reinterpret_cast<const float4*>(xrow + k + 4);
            b.w[0] = pack2_bf16(u.x, u.y); b.w[1] = pack2_bf16(u.z, u.w);
            b.w[2] = pack2_bf16(v.x, v.y); b.w[3] = pack2_bf16(v.z, v.w);
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
    }
    if (t0 + ql >= T_) return;
    if (gate) {
        const float f = 1.0f / (1.0f + expf(-gate[(size_t)(t0 + ql) * gate_stride + head]));
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] *= f;
    }
    TO* orow = out + (size_t)(t0 + ql) * o_token_stride + (size_t)head * o_head_stride + j0;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {               // registers 4 rg .. 4 rg + 3: outputs 8 rg + 4 h2 ..
        TO* dst = orow + 8 * rg + 4 * h2;
        if constexpr (sizeof(TO) == 2) {
            uint32_t* d2 = reinterpret_cast<uint32_t*>(dst);
            d2[0] = pack2_bf16(acc[4 * rg], acc[4 * rg + 1]);
            d2[1] = pack2_bf16(acc[4 * rg + 2], acc[4 * rg + 3]);
        } else {
            *reinterpret_cast<float4*>(dst) = float4{acc[4 * rg], acc[4 * rg + 1], acc[4 * rg + 2], acc[4 * rg + 3]};
        }
    }
}

template <typename TX, typename TO>
static bool headwise_mfma(const void* x, long xts, int xhs, const void* m, void* out, long ots, int ohs, int T_, int nh,
                          int n_out, int n_in, const float* gate, long gate_stride, HeadTail tail, hipStream_t stream) {
    const int ex = 16 / (int)sizeof(TX) / 2 * 2, eo = 4;       // elements that the 16-byte (32-byte) loads and the stores must start on
    if (T_ < 16 || n_in % 16 || n_out % 32 || xts % ex || xhs % ex || ots % eo || ohs % eo ||
        (uintptr_t)x % 16 || (uintptr_t)m % 16 || (uintptr_t)out % 16)
        return false;
    const dim3 grid((T_ + 31) / 32, nh, (n_out + 127) / 128);
    headwise_linear_mfma_kernel<TX, TO><<<grid, 256, 0, stream>>>((const TX*)x, xts, xhs, (const bf16_t*)m, (TO*)out, ots, ohs,
                                                                  T_, n_out, n_in, gate, gate_stride, tail);
    return true;
}

extern "C" int li_headwise_linear(const void* x, int x_dtype, long x_token_stride, int x_head_stride, const void* m, int m_dtype,
                                  void* out, int out_dtype, long o_token_stride, int o_head_stride, int T_, int nh, int n_out,
                                  int n_in, const float* gate, long gate_stride, int tail_n, int tail_split, const float* cosv,
                                  const float* sinv, hipStream_t stream) {
    if (T_ <= 0 || nh <= 0 || nh > 65535 || n_out <= 0 || n_in <= 0 || n_in > 2048 || (gate && gate_stride < nh)) return LI_ERR_SIZE;
    if (tail_n < 0 || (tail_n & 1) || (tail_n > 0 && (!cosv || !sinv || o_head_stride < n_out + tail_n))) return LI_ERR_SIZE;
    const HeadTail tail{tail_n, tail_split, cosv, sinv};
    // many tokens against bfloat16 matrices of even sizes: the matrix cores
    if (m_dtype == LI_BF16) {
        bool took = false;
        if (x_dtype == LI_F32 && out_dtype == LI_F32) took = headwise_mfma<float, float>(x, x_token_stride, x_head_stride, m, out, o_token_stride, o_head_stride, T_, nh, n_out, n_in, gate, gate_stride, tail, stream);
        else if (x_dtype == LI_F32 && out_dtype == LI_BF16) took = headwise_mfma<float, bf16_t>(x, x_token_stride, x_head_stride, m, out, o_token_stride, o_head_stride, T_, nh, n_out, n_in, gate, gate_stride, tail, stream);
        else if (x_dtype == LI_BF16 && out_dtype == LI_BF16) took = headwise_mfma<bf16_t, bf16_t>(x, x_token_stride, x_head_stride, m, out, o_token_stride, o_head_stride, T_, nh, n_out, n_in, gate, gate_stride, tail, stream);
        else if (x_dtype == LI_BF16 && out_dtype == LI_F32) took = headwise_mfma<bf16_t, float>(x, x_token_stride, x_head_stride, m, out, o_token_stride, o_head_stride, T_, nh, n_out, n_in, gate, gate_stride, tail, stream);
        if (took) return li_launch_status();
    }
    const int zs = (n_out + 63) / 64;
    const dim3 grid((T_ + HL_TOK - 1) / HL_TOK, nh, zs < 64 ? zs : 64);
    const size_t lds = (size_t)HL_TOK * n_in * 4;
#define HL_GO(TX, TM, TO)                                                                                                  \
    {                                                                                                                      \
        constexpr int E = 16 / sizeof(TM);                                                                                 \
        if (n_in % E == 0 && ((uintptr_t)m % 16) == 0)                                                                     \
            headwise_linear_kernel<TX, TM, TO, true><<<grid, 256, lds, stream>>>(                                          \
                (const TX*)x, x_token_stride, x_head_stride, (const TM*)m, (TO*)out, o_token_stride, o_head_stride, T_, n_out, n_in, gate, gate_stride, tail); \
        else                                                                                                               \
            headwise_linear_kernel<TX, TM, TO, false><<<grid, 256, lds, stream>>>(                                         \
                (const TX*)x, x_token_stride, x_head_stride, (const TM*)m, (TO*)out, o_token_stride, o_head_stride, T_, n_out, n_in, gate, gate_stride, tail); \
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
