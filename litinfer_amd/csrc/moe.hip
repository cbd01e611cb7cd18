// Routed feed-forward: the router (logits, the `top` largest, softmax over the chosen ones, and a sigmoid gate
// for a shared expert), the plan of a step (the (token, choice) pairs sorted by expert, cut into tiles of rows),
// the products of every tile's rows with its expert's matrix, and the weighted sum back into the stream.
// Nothing here returns to the host: the numbers of rows an expert gets stay on the device, and the launches are
// sized by what a step can have at most.
#include "common.h"

#define MOE_TILE 32            // rows of one expert that a tile holds
#define MOE_BIG_TILE 64        // ... where experts get hundreds of rows each (a prompt's portion): the tiles of the LDS kernel,
#define MOE_HUGE_TILE 128      // and twice that where they get still more
#define MOE_FEW_ROWS 32        // rows of a step up to which every row is a matrix-vector product of its own

// ------------------------------------------------------------------------------------------------ router
// One block a token.  logits[e] = b[e] + sum_k W[e, k] x[k] in float32 (a wave an expert, in turns); the `top`
// largest (the lower index wins a tie), weights = softmax over the chosen logits.  gate[t] = sigmoid(wg . x).
// mode 1: scores are sigmoid(logit), the choice goes by score + corr[e] inside the best groups of neighbouring
// experts, the weights are the chosen scores over their sum.  mode 2: the same with scores = softmax over ALL logits.
// Flags on top of the mode: 4: a group's score is its largest choice value (else the sum of its two largest);
// 8: the weights are the chosen scores as they are (not divided by their sum).
template <typename T> struct RouteVec;
template <> struct RouteVec<float> { static constexpr int N = 4; };
template <> struct RouteVec<bf16_t> { static constexpr int N = 8; };

// 16 bytes of a matrix row against the row in LDS
__device__ __forceinline__ float route_dot16(const float* p, const float* xs) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    return fmaf(v.x, xs[0], fmaf(v.y, xs[1], fmaf(v.z, xs[2], v.w * xs[3])));
}
__device__ __forceinline__ float route_dot16(const bf16_t* p, const float* xs) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t u[4] = {r.x, r.y, r.z, r.w};
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        s = fmaf(__uint_as_float(u[i] << 16), xs[2 * i], s);
        s = fmaf(__uint_as_float(u[i] & 0xffff0000u), xs[2 * i + 1], s);
    }
    return s;
}

template <typename TX, typename TW, int NT>
__global__ __launch_bounds__(NT) void moe_route_kernel(const TX* __restrict__ x, long x_stride, const TW* __restrict__ wr,
                                                       const float* __restrict__ br, const TW* __restrict__ wg,
                                                       int* __restrict__ idx, float* __restrict__ wt, float* __restrict__ gate,
                                                       int K, int E, int top, int vec, int mode_flags,
                                                       const float* __restrict__ corr, int groups, int keep) {
    const int mode = mode_flags & 3;
    const bool group_max = mode_flags & 4, plain_weights = mode_flags & 8;
    extern __shared__ __align__(16) float sm[];        // [K] the row, [E] the logits, [E] the scores, [groups] the groups' scores
    float* xs = sm;
    float* lg = sm + ((K + 3) & ~3);
    float* sc = lg + E;
    float* gs = sc + E;
    const int t = blockIdx.x, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const TX* row = x + (size_t)t * x_stride;
    for (int k = threadIdx.x; k < K; k += NT) xs[k] = load_as_float(row + k);
    __syncthreads();
    constexpr int VE = RouteVec<TW>::N;
    for (int e = w; e < E + (wg ? 1 : 0); e += NT / 64) {
        const TW* wrow = e < E ? wr + (size_t)e * K : wg;
        float s = 0.f;
        if (vec) {                                     // 16 bytes a lane and turn, several turns on their way
#pragma unroll 4
            for (int i = lane; i < K / VE; i += 64) s += route_dot16(wrow + (size_t)i * VE, xs + i * VE);
        } else {
            for (int k = lane; k < K; k += 64) s = fmaf(load_as_float(wrow + k), xs[k], s);
        }
        s = wave_sum(s);
        if (lane == 0) {
            if (e < E) lg[e] = s + (br ? br[e] : 0.f);
            else gate[t] = 1.0f / (1.0f + expf(-s));
        }
    }
    __syncthreads();
    if (w != 0) return;
    if (mode != 0) {
        float smx = -INFINITY, ssum = 1.f;
        if (mode == 2) {                               // softmax over all logits: the maximum and the sum, by the wave
            for (int e = lane; e < E; e += 64) smx = fmaxf(smx, lg[e]);
            smx = wave_max(smx);
            float part = 0.f;
            for (int e = lane; e < E; e += 64) part += expf(lg[e] - smx);
            ssum = wave_sum(part);
        }
        // scores s = sigmoid(logit) (mode 2: the softmax); the choice goes by s + corr among the experts of the `keep` groups (of E / groups
        // neighbours each) whose two largest choice values have the largest sum; the weights are the chosen s, normalised
        for (int e = lane; e < E; e += 64) {
            const float s = mode == 2 ? expf(lg[e] - smx) / ssum : 1.0f / (1.0f + expf(-lg[e]));
            sc[e] = s;
            lg[e] = s + (corr ? corr[e] : 0.f);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (groups > 1 && keep < groups) {
            const int per = E / groups;
            for (int g = lane; g < groups; g += 64) {
                float a = -INFINITY, b = -INFINITY;           // the largest and the second largest of the group
                for (int e = g * per; e < (g + 1) * per; ++e) {
                    const float v = lg[e];
                    if (v > a) { b = a; a = v; } else if (v > b) b = v;
                }
                gs[g] = (per > 1 && !group_max) ? a + b : a;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // a group is kept if fewer than `keep` groups come before it (a larger score, or an equal one and a lower number)
            for (int g = lane; g < groups; g += 64) {
                const float mine_s = gs[g];
                int before = 0;
                for (int o = 0; o < groups; ++o) {
                    const float v = gs[o];
                    before += (v > mine_s || (v == mine_s && o < g)) ? 1 : 0;
                }
                if (before >= keep)
                    for (int e = g * per; e < (g + 1) * per; ++e) lg[e] = -INFINITY;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
    // wave 0 picks: `top` rounds of a maximum over the logits that are left
    float chosen = 0.f, mx = 0.f, sum = 0.f;
    int mine = -1;
    for (int r = 0; r < top; ++r) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            const float v = lg[e];
            if (v > best || bi == 0x7fffffff) { best = v; bi = e; }            // (ascending e a lane: the first of equals stays)
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, LI_WAVE);
            const int oi = __shfl_xor(bi, o, LI_WAVE);
            if (oi != 0x7fffffff && (bi == 0x7fffffff || ob > best || (ob == best && oi < bi))) { best = ob; bi = oi; }
        }
        if (r == 0) mx = best;
        const float ex = mode != 0 ? sc[bi] : expf(best - mx);
        sum += ex;
        if (lane == r) { mine = bi; chosen = ex; }
        if (lane == 0) lg[bi] = -INFINITY;
        // (a wave's LDS instructions are carried out in the order of their issue: the next round reads what lane 0 wrote)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (mode != 0) sum += 1e-20f;
    if (lane < top) { idx[(size_t)t * top + lane] = mine; wt[(size_t)t * top + lane] = plain_weights ? chosen : chosen / sum; }
}

extern "C" int li_moe_route(const void* x, int x_dtype, long x_stride, const void* wr, int w_dtype, const float* br, const void* wg,
                            int* idx, float* wt, float* gate, int T, int K, int E, int top, int mode, const float* corr,
                            int groups, int keep, hipStream_t stream) {
    if (T <= 0 || K <= 0 || E <= 0 || top <= 0 || top > E || top > 64 || x_stride < K || (wg && !gate) || mode < 0 || mode > 15 || (mode & 3) == 3 ||
        groups <= 0 || keep <= 0 || keep > groups || E % groups || (size_t)(K + 2 * E + groups + 4) * 4 > 60000)
        return LI_ERR_SIZE;
    if ((mode & 3) != 0 && (long)top > (long)keep * (E / groups)) return LI_ERR_SIZE;      // more choices than the kept groups hold
    const size_t lds = (size_t)(((K + 3) & ~3) + 2 * E + groups) * 4;
    // whole 16-byte pieces of every matrix row (the gate row included)
    const int ve = w_dtype == LI_F32 ? 4 : 8;
    const int vec = K % ve == 0 && ((uintptr_t)wr % 16) == 0 && (!wg || ((uintptr_t)wg % 16) == 0);
    // few tokens: sixteen waves share a token's experts, so that a wave has one or two rows to go through
#define MR(TX, TW)                                                                                                                \
    {                                                                                                                             \
        if (T <= 128) moe_route_kernel<TX, TW, 1024><<<T, 1024, lds, stream>>>((const TX*)x, x_stride, (const TW*)wr, br, (const TW*)wg, idx, wt, gate, K, E, top, vec, mode, corr, groups, keep); \
        else moe_route_kernel<TX, TW, 256><<<T, 256, lds, stream>>>((const TX*)x, x_stride, (const TW*)wr, br, (const TW*)wg, idx, wt, gate, K, E, top, vec, mode, corr, groups, keep);           \
    }
    if (x_dtype == LI_F32 && w_dtype == LI_F32) MR(float, float)
    else if (x_dtype == LI_BF16 && w_dtype == LI_BF16) MR(bf16_t, bf16_t)
    else if (x_dtype == LI_BF16 && w_dtype == LI_F32) MR(bf16_t, float)
    else if (x_dtype == LI_F32 && w_dtype == LI_BF16) MR(float, bf16_t)
    else return LI_ERR_DTYPE;
#undef MR
    return li_launch_status();
}

// -------------------------------------------------------------------------------------------------- plan
// One block.  counts per expert, their running sum, every pair's row among its expert's rows (rows of an expert lie
// together), and the tiles: (expert, first row, rows).  plan = [n_tiles, 0, 0, 0 | tiles x 4 | ...]; row_token[row] is
// the token of a sorted row, pair_row[pair] the row of pair = token * top + choice.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ idx, int pairs, int top, int E, int* __restrict__ plan,
                                                        int max_tiles, int* __restrict__ row_token, int* __restrict__ pair_row,
                                                        int tile_rows) {
    extern __shared__ int si[];                         // [E] counts, then cursors; [E + 1] starts
    int* cnt = si;
    int* start = si + E;
    for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += 1024) {
        const int e = idx[i];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, nt = 0;
        for (int e = 0; e < E; ++e) {
            start[e] = at;
            for (int r = 0; r < cnt[e] && nt < max_tiles; r += tile_rows, ++nt) {
                int* tile = plan + 4 + 4 * nt;
                tile[0] = e; tile[1] = at + r; tile[2] = (cnt[e] - r < tile_rows) ? cnt[e] - r : tile_rows; tile[3] = 0;
            }
            at += cnt[e];
        }
        start[E] = at;
        plan[0] = nt; plan[1] = at; plan[2] = plan[3] = 0;
    }
    __syncthreads();
    // a pair's row: the next free one of its expert.  Which pair of an expert gets which of its rows depends on who
    // comes first; a row's result does not depend on where it lies
    for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += 1024) {
        const int e = idx[i];
        if (e >= 0 && e < E) {
            const int row = start[e] + atomicAdd(&cnt[e], 1);
            pair_row[i] = row;
            row_token[row] = i / top;
        } else {
            pair_row[i] = -1;
        }
    }
}

extern "C" int li_moe_plan(const int* idx, int T, int top, int E, int* plan, int max_tiles, int* row_token, int* pair_row,
                           int tile_rows, hipStream_t stream) {
    if (T <= 0 || top <= 0 || E <= 0 || E > 8000 || max_tiles <= 0 || (tile_rows != MOE_TILE && tile_rows != MOE_BIG_TILE && tile_rows != MOE_HUGE_TILE)) return LI_ERR_SIZE;
    moe_plan_kernel<<<1, 1024, (size_t)(2 * E + 1) * 4, stream>>>(idx, T * top, top, E, plan, max_tiles, row_token, pair_row, tile_rows);
    return li_launch_status();
}

// Four consecutive outputs of one row, from column `col` (a multiple of 4) on, with the activation: 0 none, 1 max(., 0)^2,
// 2 the columns are (gate, up) pairs and the two results silu(gate) * up go to columns col / 2 and col / 2 + 1;
// 3 the same pairs with g = min(gate, limit), u = clamp(up, -limit, limit) and the result g sigmoid(1.702 g) (u + 1).
__device__ __forceinline__ float moe_gated(float g, float u, int act, float limit) {
    if (act == 3) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    return u * (g / (1.0f + expf(-g)));
}

template <typename TO>
__device__ __forceinline__ void moe_store4(TO* __restrict__ row, int col, float v0, float v1, float v2, float v3, int act, float limit) {
    if (act >= 2) {
        const float o0 = moe_gated(v0, v1, act, limit), o1 = moe_gated(v2, v3, act, limit);
        TO* dst = row + (col >> 1);
        if constexpr (sizeof(TO) == 2) *reinterpret_cast<uint32_t*>(dst) = pack2_bf16(o0, o1);
        else *reinterpret_cast<float2*>(dst) = float2{o0, o1};
        return;
    }
    if (act == 1) {
        v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); v2 = fmaxf(v2, 0.f); v3 = fmaxf(v3, 0.f);
        v0 *= v0; v1 *= v1; v2 *= v2; v3 *= v3;
    }
    TO* dst = row + col;
    if constexpr (sizeof(TO) == 2) {
        uint32_t* d2 = reinterpret_cast<uint32_t*>(dst);
        d2[0] = pack2_bf16(v0, v1);
        d2[1] = pack2_bf16(v2, v3);
    } else {
        *reinterpret_cast<float4*>(dst) = float4{v0, v1, v2, v3};
    }
}

// ---------------------------------------------------------------------------------------- products by tile
// out[row, j] = act(sum_k W[e, j, k] * a[src(row), k]) for the rows of every tile, e the tile's expert; src(row) =
// row_token[row] where the rows are gathered from tokens, else the row itself.  act: 0 none, 1 max(., 0)^2, 2 the
// matrix rows come in pairs (2 j: gate, 2 j + 1: up) and out[row, j] = silu(gate) * up: half as many columns.
// General form: a block takes a tile and 64 outputs; rows and matrix rows go through LDS in float32, K in steps
// of 32; a thread owns 2 rows x 4 outputs.  Sums are float32 in the order of k.
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void moe_linear_kernel(const TA* __restrict__ a, long a_stride, const int* __restrict__ row_token,
                                                         const TW* __restrict__ w, const int* __restrict__ plan,
                                                         TO* __restrict__ out, long out_stride, int n_out, int K, int act, float limit) {
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int e = plan[4 + 4 * tile], r0 = plan[5 + 4 * tile], nr = plan[6 + 4 * tile];
    const int j0 = blockIdx.y * 64;
    __shared__ float As[MOE_TILE][33];
    __shared__ float Ws[64][33];
    __shared__ int src[MOE_TILE];
    if (threadIdx.x < MOE_TILE) {
        const int r = r0 + (threadIdx.x < nr ? threadIdx.x : 0);
        src[threadIdx.x] = row_token ? row_token[r] : r;
    }
    const int tr = threadIdx.x / 16, tc = threadIdx.x % 16;          // rows 2 tr, 2 tr + 1; outputs 2 tc + (i & 1) + 32 (i >> 1)
    float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const TW* we = w + (size_t)e * n_out * K;
    for (int k0 = 0; k0 < K; k0 += 32) {
        __syncthreads();
        for (int i = threadIdx.x; i < MOE_TILE * 32; i += 256) {
            const int r = i / 32, k = k0 + i % 32;
            As[r][i % 32] = (r < nr && k < K) ? load_as_float(a + (size_t)src[r] * a_stride + k) : 0.f;
        }
        for (int i = threadIdx.x; i < 64 * 32; i += 256) {
            const int j = j0 + i / 32, k = k0 + i % 32;
            Ws[i / 32][i % 32] = (j < n_out && k < K) ? load_as_float(we + (size_t)j * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < 32; ++k) {
            const float a0 = As[2 * tr][k], a1 = As[2 * tr + 1][k];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float wv = Ws[2 * tc + (i & 1) + 32 * (i >> 1)][k];
                acc[0][i] = fmaf(a0, wv, acc[0][i]);
                acc[1][i] = fmaf(a1, wv, acc[1][i]);
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
        const int r = 2 * tr + rr;
        if (r >= nr) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int j = j0 + 2 * tc + (i & 1) + 32 * (i >> 1);
            if (j >= n_out) continue;
            float v = acc[rr][i];
            if (act >= 2) {                            // (gate, up) pairs: i even holds the gate, i + 1 the up value
                if (i & 1) continue;
                store_from_float(out + (size_t)(r0 + r) * out_stride + (j >> 1), moe_gated(v, acc[rr][i + 1], act, limit));
                continue;
            }
            if (act == 1) { v = fmaxf(v, 0.f); v = v * v; }
            store_from_float(out + (size_t)(r0 + r) * out_stride + j, v);
        }
    }
}

// The same on the matrix cores, for bfloat16 matrices with K a multiple of 16 and n_out a multiple of 32: a wave takes
// the tile's 32 rows and 32 outputs and works on the transposed tile (outputs x rows), so that both operands are
// 16-byte pieces of rows as they lie in memory and a lane ends with four consecutive outputs of its row.
typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x16 __attribute__((ext_vector_type(16)));
union moe_frag8 { uint4 raw; uint32_t w[4]; moe_bf16x8 v; };

template <typename TA, typename TO>
__global__ __launch_bounds__(256) void moe_linear_mfma_kernel(const TA* __restrict__ a, long a_stride, const int* __restrict__ row_token,
                                                              const bf16_t* __restrict__ w, const int* __restrict__ plan,
                                                              TO* __restrict__ out, long out_stride, int n_out, int K, int act, float limit) {
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int e = plan[4 + 4 * tile], r0 = plan[5 + 4 * tile], nr = plan[6 + 4 * tile];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, ql = lane & 31, h2 = lane >> 5;
    const int j0 = (blockIdx.y * 4 + wv) * 32;
    if (j0 >= n_out) return;
    const int r = r0 + (ql < nr ? ql : 0);
    const int srow = row_token ? row_token[r] : r;
    const TA* arow = a + (size_t)srow * a_stride + 8 * h2;
    const bf16_t* mrow = w + ((size_t)e * n_out + j0 + ql) * K + 8 * h2;
    moe_f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    for (int k = 0; k < K; k += 16) {
        moe_frag8 fa, fb;
        fa.raw = *reinterpret_cast<const uint4*>(mrow + k);
        if constexpr (sizeof(TA) == 2) {
            fb.raw = *reinterpret_cast<const uint4*>(arow + k);
        } else {
            const float4 u = *reinterpret_cast<const float4*>(arow + k);
            const float4 v = *reinterpret_cast<const float4*>(arow + k + 4);
            fb.w[0] = pack2_bf16(u.x, u.y); fb.w[1] = pack2_bf16(u.z, u.w);
            fb.w[2] = pack2_bf16(v.x, v.y); fb.w[3] = pack2_bf16(v.z, v.w);
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.v, fb.v, acc, 0, 0, 0);
    }
    if (ql >= nr) return;
    TO* orow = out + (size_t)(r0 + ql) * out_stride;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg)                     // registers 4 rg .. 4 rg + 3: outputs 8 rg + 4 h2 ..
        moe_store4(orow, j0 + 8 * rg + 4 * h2, acc[4 * rg], acc[4 * rg + 1], acc[4 * rg + 2], acc[4 * rg + 3], act, limit);
}

// The wider form, for K a multiple of 32: a wave takes the tile's 32 rows and 128 outputs (four accumulators that
// share the rows' operand), K in steps of 32 with the next step's ten loads asked for before this step's eight
// matrix products.  KSPLIT = 1: the four waves of a block take 512 outputs side by side (many rows: a prompt).
// KSPLIT = 4: they take the same 128 outputs and a quarter of K each and add up through LDS, so that the few tiles
// of a decoding step, each of which streams its expert's whole matrix, are spread over four times the waves.
template <typename TA>
__device__ __forceinline__ void moe_load_rows(moe_frag8& f, const TA* p) {
    if constexpr (sizeof(TA) == 2) {
        f.raw = *reinterpret_cast<const uint4*>(p);
    } else {
        const float4 u = *reinterpret_cast<const float4*>(p);
        const float4 v = *reinterpret_cast<const float4*>(p + 4);
        f.w[0] = pack2_bf16(u.x, u.y); f.w[1] = pack2_bf16(u.z, u.w);
        f.w[2] = pack2_bf16(v.x, v.y); f.w[3] = pack2_bf16(v.z, v.w);
    }
}

template <typename TA, typename TO, int KSPLIT>
__global__ __launch_bounds__(256) void moe_linear_wide_kernel(const TA* __restrict__ a, long a_stride, const int* __restrict__ row_token,
                                                              const bf16_t* __restrict__ w, const int* __restrict__ plan,
                                                              TO* __restrict__ out, long out_stride, int n_out, int K, int act, float limit,
                                                              int max_tiles) {
    int tile = blockIdx.x, cb = blockIdx.y;
    if (KSPLIT == 1) {
        // Many tiles: the grid is one row of blocks, which the chip deals out to its eight XCDs in turn.  Eight tiles
        // that follow each other (mostly rows of one expert) against the same columns go to ONE XCD, next to each other
        // in time, so that the expert's matrix comes into that XCD's L2 once for them and not once for each XCD.
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        const int item = (((idx >> 3) << 3) + xcd) * 8 + (idx & 7);
        const int tiles = max_tiles;
        cb = item / tiles;
        tile = item % tiles;
    }
    if (tile >= plan[0]) return;
    const int e = plan[4 + 4 * tile], r0 = plan[5 + 4 * tile], nr = plan[6 + 4 * tile];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, ql = lane & 31, h2 = lane >> 5;
    const int j0 = (KSPLIT == 1 ? cb * 4 + wv : cb) * 128;
    if (KSPLIT == 1 && j0 >= n_out) return;
    int nf = (n_out - j0) / 32;                        // column fragments of 32 that exist (n_out is a multiple of 32)
    if (nf > 4) nf = 4;
    int k0 = 0, k1 = K;
    if (KSPLIT > 1) {
        const int per = ((K / 32 + KSPLIT - 1) / KSPLIT) * 32;
        k0 = wv * per;
        k1 = k0 + per < K ? k0 + per : K;
    }
    const int r = r0 + (ql < nr ? ql : 0);
    const TA* arow = a + (size_t)(row_token ? row_token[r] : r) * a_stride + 8 * h2;
    const bf16_t* mrow[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) mrow[f] = w + ((size_t)e * n_out + j0 + 32 * (f < nf ? f : 0) + ql) * K + 8 * h2;
    moe_f32x16 acc[4];
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[f][i] = 0.f;
    moe_frag8 ca[2], cw[4][2], na[2], nw[4][2];
    if (k0 < k1) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            moe_load_rows<TA>(ca[s2], arow + k0 + 16 * s2);
#pragma unroll
            for (int f = 0; f < 4; ++f) cw[f][s2].raw = *reinterpret_cast<const uint4*>(mrow[f] + k0 + 16 * s2);
        }
    }
    for (int k = k0; k < k1; k += 32) {
        const int kn = k + 32 < k1 ? k + 32 : k;       // (the last turn asks for its own step again: no branch around the loads)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            moe_load_rows<TA>(na[s2], arow + kn + 16 * s2);
#pragma unroll
            for (int f = 0; f < 4; ++f) nw[f][s2].raw = *reinterpret_cast<const uint4*>(mrow[f] + kn + 16 * s2);
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int f = 0; f < 4; ++f) acc[f] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cw[f][s2].v, ca[s2].v, acc[f], 0, 0, 0);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            ca[s2] = na[s2];
#pragma unroll
            for (int f = 0; f < 4; ++f) cw[f][s2] = nw[f][s2];
        }
    }
    int f_lo = 0, f_hi = nf;
    if (KSPLIT > 1) {
        // the four waves' sums meet in LDS; wave f then owns column fragment f
        __shared__ float red[KSPLIT][4][16][64];
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int i = 0; i < 16; ++i) red[wv][f][i][lane] = acc[f][i];
        __syncthreads();
        if (wv >= nf) return;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float t = 0.f;
#pragma unroll
            for (int src = 0; src < KSPLIT; ++src) t += red[src][wv][i][lane];
            acc[0][i] = t;
        }
        f_lo = wv;
        f_hi = wv + 1;
    }
    if (ql >= nr) return;
    TO* orow = out + (size_t)(r0 + ql) * out_stride;
    for (int f = f_lo; f < f_hi; ++f) {
        const moe_f32x16 c = KSPLIT > 1 ? acc[0] : (f == 0 ? acc[0] : f == 1 ? acc[1] : f == 2 ? acc[2] : acc[3]);
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)                 // registers 4 rg .. 4 rg + 3: outputs 32 f + 8 rg + 4 h2 ..
            moe_store4(orow, j0 + 32 * f + 8 * rg + 4 * h2, c[4 * rg], c[4 * rg + 1], c[4 * rg + 2], c[4 * rg + 3], act, limit);
    }
}

// A handful of rows in all (a decoding step of few requests): every tile streams its expert's matrix for one or two
// rows, so the product is a matrix-vector product a row.  A wave owns four outputs and walks their matrix rows in
// 16-byte pieces, 64 lanes side by side along K (a kilobyte of a row at a time, all four rows' pieces asked for
// together), against up to four of the tile's rows at a time; sums in float32, lanes added up at the end.
#define MR_OUT 4
#define MR_ROWS 4

template <typename TO>
__global__ __launch_bounds__(256) void moe_linear_rows_kernel(const bf16_t* __restrict__ a, long a_stride, const int* __restrict__ row_token,
                                                              const bf16_t* __restrict__ w, const int* __restrict__ plan,
                                                              TO* __restrict__ out, long out_stride, int n_out, int K, int act, float limit) {
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int e = plan[4 + 4 * tile], r0 = plan[5 + 4 * tile], nr = plan[6 + 4 * tile];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int j0 = (blockIdx.y * 4 + wv) * MR_OUT;
    if (j0 >= n_out) return;
    const bf16_t* wrow[MR_OUT];
#pragma unroll
    for (int j = 0; j < MR_OUT; ++j) wrow[j] = w + ((size_t)e * n_out + (j0 + j < n_out ? j0 + j : n_out - 1)) * K;
    for (int rc = 0; rc < nr; rc += MR_ROWS) {
        const bf16_t* xrow[MR_ROWS];
#pragma unroll
        for (int r = 0; r < MR_ROWS; ++r) {
            const int row = r0 + (rc + r < nr ? rc + r : nr - 1);
            xrow[r] = a + (size_t)(row_token ? row_token[row] : row) * a_stride;
        }
        float acc[MR_OUT][MR_ROWS];
#pragma unroll
        for (int j = 0; j < MR_OUT; ++j)
#pragma unroll
            for (int r = 0; r < MR_ROWS; ++r) acc[j][r] = 0.f;
        for (int i = lane; i < K / 8; i += 64) {
            uint4 wp[MR_OUT], xp[MR_ROWS];
#pragma unroll
            for (int j = 0; j < MR_OUT; ++j) wp[j] = *reinterpret_cast<const uint4*>(wrow[j] + 8 * i);
#pragma unroll
            for (int r = 0; r < MR_ROWS; ++r) xp[r] = *reinterpret_cast<const uint4*>(xrow[r] + 8 * i);
            float xf[MR_ROWS][8];
#pragma unroll
            for (int r = 0; r < MR_ROWS; ++r) {
                const uint32_t u[4] = {xp[r].x, xp[r].y, xp[r].z, xp[r].w};
#pragma unroll
                for (int q = 0; q < 4; ++q) { xf[r][2 * q] = __uint_as_float(u[q] << 16); xf[r][2 * q + 1] = __uint_as_float(u[q] & 0xffff0000u); }
            }
#pragma unroll
            for (int j = 0; j < MR_OUT; ++j) {
                const uint32_t u[4] = {wp[j].x, wp[j].y, wp[j].z, wp[j].w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float lo = __uint_as_float(u[q] << 16), hi = __uint_as_float(u[q] & 0xffff0000u);
#pragma unroll
                    for (int r = 0; r < MR_ROWS; ++r) acc[j][r] = fmaf(hi, xf[r][2 * q + 1], fmaf(lo, xf[r][2 * q], acc[j][r]));
                }
            }
        }
#pragma unroll
        for (int j = 0; j < MR_OUT; ++j)
#pragma unroll
            for (int r = 0; r < MR_ROWS; ++r) acc[j][r] = wave_sum(acc[j][r]);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < MR_ROWS; ++r) {
                if (rc + r >= nr) continue;
                TO* orow = out + (size_t)(r0 + rc + r) * out_stride;
                if (act >= 2) {                        // (gate, up) pairs: n_out is even and j0 a multiple of 4
#pragma unroll
                    for (int j = 0; j < MR_OUT; j += 2)
                        if (j0 + j < n_out) store_from_float(orow + ((j0 + j) >> 1), moe_gated(acc[j][r], acc[j + 1][r], act, limit));
                    continue;
                }
#pragma unroll
                for (int j = 0; j < MR_OUT; ++j) {
                    if (j0 + j >= n_out) continue;
                    float v = acc[j][r];
                    if (act == 1) { v = fmaxf(v, 0.f); v = v * v; }
                    store_from_float(orow + j0 + j, v);
                }
            }
        }
    }
}

// Many rows an expert (tiles of up to 64 rows): a block takes a tile and 128 outputs, K in steps of 32 through LDS, so
// that a matrix row that came from memory serves 64 rows and a token's row 128 outputs; its four waves are two by two,
// each with 32 rows x 64 outputs (two accumulators).  The block is small on purpose: five or more of them share a compute
// unit, and while one waits for its next pieces (they wait in registers while this step is multiplied) or at its
// barriers, the others multiply.  bfloat16 rows and matrices; the same transposed tiles (outputs x rows) as above.
#define MB_COLS 128
#define MB_K 32                // k-values a step (64 bytes of a row: with 128 a block's LDS doubles and half as many blocks share a compute unit: 298 against 210 us)
#define MB_DEPTH 2             // steps whose pieces wait in registers (four: no faster)
#define MB_LD (MB_K + 8)       // elements of an LDS row: 8 of padding (144 bytes: the 16-byte reads of 16 lanes spread over the banks)

template <typename TO, int RF>      // RF: row fragments of 32 a wave (1: tiles of 64 rows, 2: of 128)
__global__ __launch_bounds__(256) void moe_linear_lds_kernel(const bf16_t* __restrict__ a, long a_stride, const int* __restrict__ row_token,
                                                             const bf16_t* __restrict__ w, const int* __restrict__ plan,
                                                             TO* __restrict__ out, long out_stride, int n_out, int K, int act, float limit,
                                                             int max_tiles) {
    constexpr int MB_ROWS = 64 * RF;
    __shared__ __align__(16) uint16_t As[MB_ROWS * MB_LD];
    __shared__ __align__(16) uint16_t Ws[MB_COLS * MB_LD];
    __shared__ int src[MB_ROWS];
    // (eight tiles that follow each other against the same columns go to one XCD: see the wide kernel)
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int item = (((idx >> 3) << 3) + xcd) * 8 + (idx & 7);
    const int cb = item / max_tiles, tile = item % max_tiles;
    if (tile >= plan[0] || cb * MB_COLS >= n_out) return;
    const int e = plan[4 + 4 * tile], r0 = plan[5 + 4 * tile], nr = plan[6 + 4 * tile];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, ql = lane & 31, h2 = lane >> 5;
    const int j0 = cb * MB_COLS;
    if (tid < MB_ROWS) {
        const int r = r0 + (tid < nr ? tid : nr - 1);
        src[tid] = row_token ? row_token[r] : r;
    }
    __syncthreads();
    // what a thread brings in a step: 16-byte pieces, MB_K / 8 to a row: NA of token rows, NW of matrix rows
    constexpr int PP = MB_K / 8, RP = 256 / PP, NA = MB_ROWS / RP, NW = MB_COLS / RP;
    const int prow = tid / PP, part = tid % PP;
    const bf16_t* ga[NA];
    const bf16_t* gw[NW];
    int la[NA], lw[NW];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int row = prow + RP * i;
        ga[i] = a + (size_t)src[row] * a_stride + 8 * part;
        la[i] = row * MB_LD + 8 * part;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const int row = prow + RP * i;
        const int j = j0 + row < n_out ? j0 + row : n_out - 1;
        gw[i] = w + ((size_t)e * n_out + j) * K + 8 * part;
        lw[i] = row * MB_LD + 8 * part;
    }
    const int wr = wv >> 1, wc = wv & 1;               // the wave's 32 * RF rows and 64 outputs
    moe_f32x16 acc[RF][2];
#pragma unroll
    for (int rf = 0; rf < RF; ++rf)
#pragma unroll
        for (int cf = 0; cf < 2; ++cf)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[rf][cf][i] = 0.f;
    // the pieces of the next MB_DEPTH steps wait in registers: a step's pieces are asked for that many steps before they go to LDS
    uint4 ra[MB_DEPTH][NA], rw[MB_DEPTH][NW];
    const int last = K - MB_K;
#pragma unroll
    for (int d = 0; d < MB_DEPTH; ++d) {
        const int kd = d * MB_K < last ? d * MB_K : last;
#pragma unroll
        for (int i = 0; i < NA; ++i) ra[d][i] = *reinterpret_cast<const uint4*>(ga[i] + kd);
#pragma unroll
        for (int i = 0; i < NW; ++i) rw[d][i] = *reinterpret_cast<const uint4*>(gw[i] + kd);
    }
    for (int k = 0; k < K; k += MB_K) {
        __syncthreads();                               // the step before has been read
#pragma unroll
        for (int i = 0; i < NA; ++i) *reinterpret_cast<uint4*>(&As[la[i]]) = ra[0][i];
#pragma unroll
        for (int i = 0; i < NW; ++i) *reinterpret_cast<uint4*>(&Ws[lw[i]]) = rw[0][i];
        __syncthreads();
        const int kn = k + MB_DEPTH * MB_K < last ? k + MB_DEPTH * MB_K : last;      // (past the end: the last step again, no branch around the loads)
#pragma unroll
        for (int i = 0; i < NA; ++i) {
#pragma unroll
            for (int d = 0; d + 1 < MB_DEPTH; ++d) ra[d][i] = ra[d + 1][i];
            ra[MB_DEPTH - 1][i] = *reinterpret_cast<const uint4*>(ga[i] + kn);
        }
#pragma unroll
        for (int i = 0; i < NW; ++i) {
#pragma unroll
            for (int d = 0; d + 1 < MB_DEPTH; ++d) rw[d][i] = rw[d + 1][i];
            rw[MB_DEPTH - 1][i] = *reinterpret_cast<const uint4*>(gw[i] + kn);
        }
#pragma unroll
        for (int s2 = 0; s2 < MB_K / 16; ++s2) {
            moe_frag8 fa[RF], fw[2];
#pragma unroll
            for (int rf = 0; rf < RF; ++rf)
                fa[rf].raw = *reinterpret_cast<const uint4*>(&As[(32 * RF * wr + 32 * rf + ql) * MB_LD + 16 * s2 + 8 * h2]);
#pragma unroll
            for (int cf = 0; cf < 2; ++cf)
                fw[cf].raw = *reinterpret_cast<const uint4*>(&Ws[(64 * wc + 32 * cf + ql) * MB_LD + 16 * s2 + 8 * h2]);
#pragma unroll
            for (int rf = 0; rf < RF; ++rf)
#pragma unroll
                for (int cf = 0; cf < 2; ++cf)
                    acc[rf][cf] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[cf].v, fa[rf].v, acc[rf][cf], 0, 0, 0);
        }
    }
#pragma unroll
    for (int rf = 0; rf < RF; ++rf) {
        const int row = 32 * RF * wr + 32 * rf + ql;
        if (row >= nr) continue;
        TO* orow = out + (size_t)(r0 + row) * out_stride;
#pragma unroll
        for (int cf = 0; cf < 2; ++cf) {
            if (j0 + 64 * wc + 32 * cf >= n_out) continue;
#pragma unroll
            for (int rg = 0; rg < 4; ++rg)             // registers 4 rg .. 4 rg + 3: outputs 32 cf + 8 rg + 4 h2 ..
                moe_store4(orow, j0 + 64 * wc + 32 * cf + 8 * rg + 4 * h2, acc[rf][cf][4 * rg], acc[rf][cf][4 * rg + 1],
                           acc[rf][cf][4 * rg + 2], acc[rf][cf][4 * rg + 3], act, limit);
        }
    }
}

// 1 if tiles of MOE_BIG_TILE rows have a kernel for these operands
extern "C" int li_moe_linear_big_takes(int a_dtype, int w_dtype, int n_out, int K) {
    return a_dtype == LI_BF16 && w_dtype == LI_BF16 && K % MB_K == 0 && n_out % 32 == 0;
}

extern "C" int li_moe_linear(const void* a, int a_dtype, long a_stride, const int* row_token, const void* w, int w_dtype,
                             const int* plan, int max_tiles, void* out, int out_dtype, long out_stride, int n_out, int K, int act, float limit,
                             int tile_rows, int rows, hipStream_t stream) {
    if (max_tiles <= 0 || n_out <= 0 || K <= 0 || a_stride < K || act < 0 || act > 3 || out_stride < (act >= 2 ? n_out / 2 : n_out) ||
        (act >= 2 && (n_out & 1)))
        return LI_ERR_SIZE;
    if (tile_rows == MOE_BIG_TILE || tile_rows == MOE_HUGE_TILE) {
        if (!li_moe_linear_big_takes(a_dtype, w_dtype, n_out, K) || a_stride % 8 || out_stride % 4 ||
            ((uintptr_t)a | (uintptr_t)w | (uintptr_t)out) % 16)
            return LI_ERR_SIZE;
        const dim3 line((unsigned)((((long)max_tiles * ((n_out + MB_COLS - 1) / MB_COLS) + 63) / 64) * 64));
#define ML(TO, RF) moe_linear_lds_kernel<TO, RF><<<line, 256, 0, stream>>>((const bf16_t*)a, a_stride, row_token, (const bf16_t*)w, plan, (TO*)out, out_stride, n_out, K, act, limit, max_tiles)
        const bool huge = tile_rows == MOE_HUGE_TILE;
        if (out_dtype == LI_BF16) { if (huge) ML(bf16_t, 2); else ML(bf16_t, 1); }
        else if (out_dtype == LI_F32) { if (huge) ML(float, 2); else ML(float, 1); }
        else return LI_ERR_DTYPE;
#undef ML
        return li_launch_status();
    }
    if (tile_rows != MOE_TILE) return LI_ERR_SIZE;
    // a handful of rows in all: a matrix-vector product a row (each tile streams its expert's matrix anyway)
    if (rows <= MOE_FEW_ROWS && a_dtype == LI_BF16 && w_dtype == LI_BF16 && K % 8 == 0 && a_stride % 8 == 0 &&
        ((uintptr_t)a | (uintptr_t)w) % 16 == 0 && (out_dtype == LI_BF16 || out_dtype == LI_F32)) {
        const dim3 grid(max_tiles, (n_out + 4 * MR_OUT - 1) / (4 * MR_OUT));
        if (out_dtype == LI_BF16)
            moe_linear_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, row_token, (const bf16_t*)w, plan, (bf16_t*)out, out_stride, n_out, K, act, limit);
        else
            moe_linear_rows_kernel<float><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, row_token, (const bf16_t*)w, plan, (float*)out, out_stride, n_out, K, act, limit);
        return li_launch_status();
    }
    if (w_dtype == LI_BF16 && K % 16 == 0 && n_out % 32 == 0 && a_stride % 8 == 0 && out_stride % 4 == 0 &&
        ((uintptr_t)a | (uintptr_t)w | (uintptr_t)out) % 16 == 0 && (a_dtype == LI_BF16 || a_dtype == LI_F32)) {
        // few tiles (a decoding step: each streams its expert's whole matrix): K in quarters over a block's waves
        const bool wide = K % 32 == 0, split = wide && max_tiles <= 128 && K >= 256;
        const dim3 grid(max_tiles, (n_out + 127) / 128);
        const dim3 line((unsigned)((((long)max_tiles * ((n_out + 511) / 512) + 63) / 64) * 64));       // whole rounds of eight tiles over eight XCDs
#define MM(TA, TO)                                                                                                                 \
    {                                                                                                                              \
        if (split) moe_linear_wide_kernel<TA, TO, 4><<<grid, 256, 0, stream>>>((const TA*)a, a_stride, row_token, (const bf16_t*)w, plan, (TO*)out, out_stride, n_out, K, act, limit, max_tiles); \
        else if (wide) moe_linear_wide_kernel<TA, TO, 1><<<line, 256, 0, stream>>>((const TA*)a, a_stride, row_token, (const bf16_t*)w, plan, (TO*)out, out_stride, n_out, K, act, limit, max_tiles); \
        else moe_linear_mfma_kernel<TA, TO><<<grid, 256, 0, stream>>>((const TA*)a, a_stride, row_token, (const bf16_t*)w, plan, (TO*)out, out_stride, n_out, K, act, limit); \
    }
        if (a_dtype == LI_BF16 && out_dtype == LI_BF16) MM(bf16_t, bf16_t)
        else if (a_dtype == LI_BF16 && out_dtype == LI_F32) MM(bf16_t, float)
        else if (a_dtype == LI_F32 && out_dtype == LI_BF16) MM(float, bf16_t)
        else if (a_dtype == LI_F32 && out_dtype == LI_F32) MM(float, float)
        else return LI_ERR_DTYPE;
#undef MM
        return li_launch_status();
    }
    const dim3 grid(max_tiles, (n_out + 63) / 64);
#define ML(TA, TW, TO) moe_linear_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>((const TA*)a, a_stride, row_token, (const TW*)w, plan, (TO*)out, out_stride, n_out, K, act, limit)
    if (a_dtype == LI_F32 && w_dtype == LI_F32 && out_dtype == LI_F32) ML(float, float, float);
    else if (a_dtype == LI_BF16 && w_dtype == LI_BF16 && out_dtype == LI_BF16) ML(bf16_t, bf16_t, bf16_t);
    else if (a_dtype == LI_BF16 && w_dtype == LI_BF16 && out_dtype == LI_F32) ML(bf16_t, bf16_t, float);
    else if (a_dtype == LI_F32 && w_dtype == LI_BF16 && out_dtype == LI_F32) ML(float, bf16_t, float);
    else if (a_dtype == LI_F32 && w_dtype == LI_BF16 && out_dtype == LI_BF16) ML(float, bf16_t, bf16_t);
    else return LI_ERR_DTYPE;
#undef ML
    return li_launch_status();
}

// ----------------------------------------------------------------------------------------------- the sum
// x[t, :] += sum_c wt[t, c] * yrow[pair_row[t * top + c], :] (in the order of c) + gate[t] * shared[t, :].  A choice
// idx[t, c] >= experts (where `ident` is given) is an IDENTITY expert: its output is the token's input row ident[t, :].
template <typename TI>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, long x_stride, const float* __restrict__ yrows,
                                                          long y_stride, const int* __restrict__ pair_row, const float* __restrict__ wt,
                                                          const float* __restrict__ gate, const float* __restrict__ shared_out,
                                                          long s_stride, int H, int top, const int* __restrict__ idx, int experts,
                                                          const TI* __restrict__ ident, long i_stride) {
    const int t = blockIdx.x;
    for (int j = blockIdx.y * 256 + threadIdx.x; j < H; j += gridDim.y * 256) {
        float s = 0.f;
        for (int c = 0; c < top; ++c) {
            const int row = pair_row[(size_t)t * top + c];
            if (row >= 0) s = fmaf(wt[(size_t)t * top + c], yrows[(size_t)row * y_stride + j], s);
            else if (ident && idx[(size_t)t * top + c] >= experts)
                s = fmaf(wt[(size_t)t * top + c], load_as_float(ident + (size_t)t * i_stride + j), s);
        }
        if (shared_out) s = fmaf(gate ? gate[t] : 1.f, shared_out[(size_t)t * s_stride + j], s);
        x[(size_t)t * x_stride + j] += s;
    }
}

extern "C" int li_moe_combine(float* x, long x_stride, const float* yrows, long y_stride, const int* pair_row, const float* wt,
                              const float* gate, const float* shared_out, long s_stride, int T, int H, int top,
                              const int* idx, int experts, const void* ident, int ident_dtype, long i_stride, hipStream_t stream) {
    if (T <= 0 || H <= 0 || top <= 0 || x_stride < H || y_stride < H || (shared_out && s_stride < H) ||
        (ident && (!idx || i_stride < H || experts < 0)))
        return LI_ERR_SIZE;
    int ys = (H + 255) / 256;
    if (ys > 64) ys = 64;
    if (ident && ident_dtype == LI_BF16)
        moe_combine_kernel<bf16_t><<<dim3(T, ys), 256, 0, stream>>>(x, x_stride, yrows, y_stride, pair_row, wt, gate, shared_out, s_stride, H, top,
                                                                    idx, experts, (const bf16_t*)ident, i_stride);
    else if (!ident || ident_dtype == LI_F32)
        moe_combine_kernel<float><<<dim3(T, ys), 256, 0, stream>>>(x, x_stride, yrows, y_stride, pair_row, wt, gate, shared_out, s_stride, H, top,
                                                                   idx, experts, (const float*)ident, i_stride);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}
