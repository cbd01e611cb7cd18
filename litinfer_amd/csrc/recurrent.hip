// Kernels of recurrent mixers whose state has a fixed size per request: a short causal convolution
// per channel with its tail of past inputs, the selective state-space recurrence
//   S_t = a_t S_{t-1} + dt_t B_t x_t^T,  y_t = S_t^T C_t + D x_t,  a_t = exp(-exp(A_log) dt_t),
// (with `fixed_a`: a_t = fixed_a[head] and dt_t = fixed_dt for every token, a retention with a decay a head),
// the gated delta rule, and the gated RMS norm in groups of columns behind them.  Everything here is float32: inputs, decays,
// step sizes, the state and the sums; only the normed output is rounded to the activations' type.
#include "common.h"

// ------------------------------------------------------------------------------------ causal convolution
// out[t, c] = silu(b[c] + sum_j w[c, j] * u[t - (taps - 1 - j), c]): the last column of w multiplies the
// current token.  Inputs before the first token of the step's portion come from the request's tail
// [slots, taps - 1, C] (its last taps - 1 inputs, zeros for a new request).
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    const float* __restrict__ u, long u_stride, int C, int taps, const float* __restrict__ w, const float* __restrict__ b,
    const float* __restrict__ tail, const int* __restrict__ seg_of_token, const int* __restrict__ q_start,
    const int* __restrict__ slots, float* __restrict__ out, long out_stride, float* __restrict__ tail_out) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int seg = seg_of_token[t], i = t - q_start[seg], slot = slots[seg];
    float acc = b ? b[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j, li = i - back;
        const float v = li >= 0 ? u[(size_t)(t - back) * u_stride + c]
                                : tail[((size_t)slot * (taps - 1) + (taps - 1 + li)) * C + c];
        acc = fmaf(w[(size_t)c * taps + j], v, acc);
        // every request brings one token (tail_out is given then): the thread owns the request's channel and moves
        // its tail up by one as it goes (it has read place j, and will read place j + 1 next)
        if (tail_out && j > 0) tail_out[((size_t)slot * (taps - 1) + (j - 1)) * C + c] = v;
    }
    out[(size_t)t * out_stride + c] = acc / (1.0f + expf(-acc));
}

// The same for many tokens with four neighbouring channels a thread (channels, strides and addresses in multiples of
// four floats): 16-byte loads and stores; the taps' weights of the four channels lie one after the other.
template <int TAPS>
__global__ __launch_bounds__(256) void causal_conv_silu_vec_kernel(
    const float* __restrict__ u, long u_stride, int C, const float* __restrict__ w, const float* __restrict__ b,
    const float* __restrict__ tail, const int* __restrict__ seg_of_token, const int* __restrict__ q_start,
    const int* __restrict__ slots, float* __restrict__ out, long out_stride) {
    const int t = blockIdx.x, c = 4 * (blockIdx.y * 256 + threadIdx.x);
    if (c >= C) return;
    const int seg = seg_of_token[t], i = t - q_start[seg], slot = slots[seg];
    float4 acc = b ? *reinterpret_cast<const float4*>(b + c) : float4{0.f, 0.f, 0.f, 0.f};
    float wv[4][TAPS];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int j = 0; j < TAPS; ++j) wv[k][j] = w[(size_t)(c + k) * TAPS + j];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
        const int back = TAPS - 1 - j, li = i - back;
        const float4 v = *reinterpret_cast<const float4*>(li >= 0 ? u + (size_t)(t - back) * u_stride + c
                                                                  : tail + ((size_t)slot * (TAPS - 1) + (TAPS - 1 + li)) * C + c);
        acc.x = fmaf(wv[0][j], v.x, acc.x);
        acc.y = fmaf(wv[1][j], v.y, acc.y);
        acc.z = fmaf(wv[2][j], v.z, acc.z);
        acc.w = fmaf(wv[3][j], v.w, acc.w);
    }
    *reinterpret_cast<float4*>(out + (size_t)t * out_stride + c) =
        float4{acc.x / (1.0f + expf(-acc.x)), acc.y / (1.0f + expf(-acc.y)), acc.z / (1.0f + expf(-acc.z)), acc.w / (1.0f + expf(-acc.w))};
}

// The tail after the step: the last taps - 1 inputs of the request, those of this portion and, where it is
// shorter than that, what is left of the old tail.  A thread owns a (request, channel) and goes upwards, so
// it never reads what it has written.
__global__ __launch_bounds__(256) void conv_tail_update_kernel(
    const float* __restrict__ u, long u_stride, int C, int taps, float* __restrict__ tail,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ slots) {
    const int seg = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int L = q_len[seg], t0 = q_start[seg];
    float* mine = tail + (size_t)slots[seg] * (taps - 1) * C + c;
    for (int r = 0; r < taps - 1; ++r) {
        const int li = L - (taps - 1) + r;
        mine[(size_t)r * C] = li >= 0 ? u[(size_t)(t0 + li) * u_stride + c] : mine[(size_t)(r + L) * C];
    }
}

extern "C" int li_causal_conv_silu(const float* u, long u_stride, int C, int taps, const float* w, const float* b, float* tail,
                                   const int* seg_of_token, const int* q_start, const int* q_len, const int* slots,
                                   float* out, long out_stride, int T, int segs, int max_q_len, hipStream_t stream) {
    if (T <= 0 || segs <= 0 || C <= 0 || taps <= 0 || taps > 64 || u_stride < C || out_stride < C || max_q_len <= 0) return LI_ERR_SIZE;
    const dim3 grid(T, (C + 255) / 256);
    const bool single = max_q_len == 1 && taps > 1;            // a decoding step: one kernel does both
    const bool vec = !single && T >= 64 && taps >= 2 && taps <= 4 && C % 4 == 0 && u_stride % 4 == 0 && out_stride % 4 == 0 &&
                     ((uintptr_t)u | (uintptr_t)out | (uintptr_t)tail | (uintptr_t)b) % 16 == 0;
    const dim3 grid4(T, (C / 4 + 255) / 256);
    if (vec && taps == 2)
        causal_conv_silu_vec_kernel<2><<<grid4, 256, 0, stream>>>(u, u_stride, C, w, b, tail, seg_of_token, q_start, slots, out, out_stride);
    else if (vec && taps == 3)
        causal_conv_silu_vec_kernel<3><<<grid4, 256, 0, stream>>>(u, u_stride, C, w, b, tail, seg_of_token, q_start, slots, out, out_stride);
    else if (vec)
        causal_conv_silu_vec_kernel<4><<<grid4, 256, 0, stream>>>(u, u_stride, C, w, b, tail, seg_of_token, q_start, slots, out, out_stride);
    else
        causal_conv_silu_kernel<<<grid, 256, 0, stream>>>(u, u_stride, C, taps, w, b, tail, seg_of_token, q_start, slots, out, out_stride,
                                                          single ? tail : nullptr);
    if (taps > 1 && !single) {
        const dim3 g2(segs, (C + 255) / 256);
        conv_tail_update_kernel<<<g2, 256, 0, stream>>>(u, u_stride, C, taps, tail, q_start, q_len, slots);
    }
    return li_launch_status();
}

// ------------------------------------------------------------------------------------ state-space recurrence
// A column p of a head's state (its N values) evolves by itself, given x_t[p] and the head's a_t, dt_t, B_t,
// C_t.  A lane owns NR state values of one column in registers: lane = column * NS + slice, the slices of a
// column are NS neighbouring lanes that add their shares of y up.  A wave is 64 / NS columns of one head; the
// four waves of a block are heads (or column ranges) of ONE group and share its B_t and C_t, which lie in LDS
// for SSM_TB tokens at a time beside each wave's x_t, dt_t and a_t.
//
// A step's portion of a request is cut into chunks of Q tokens that run side by side:
//   MODE 1: the state that a chunk alone builds up from zero, and the product of its decays;
//   the carry kernel: the state with which every chunk begins, chunk after chunk;
//   MODE 0: the recurrence itself from that state, with the outputs; the last chunk leaves the request's state.
// A portion of at most Q tokens (a decoding step) is MODE 0 alone, from the request's state.
#define SSM_TB 16
#define SSM_WAVES 4

__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <int NR, int NS, int MODE>
__global__ __launch_bounds__(64 * SSM_WAVES) void ssm_scan_kernel(
    const float* __restrict__ xbc, long xbc_stride, const float* __restrict__ dt_raw, long dt_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dw,
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ q_start, const int* __restrict__ q_len,
    const int* __restrict__ chunk_seg, const int* __restrict__ chunk_idx, float* __restrict__ carry, float* __restrict__ decay,
    float* __restrict__ y, long y_stride, int heads, int vdim, int N, int G, int Q, const float* __restrict__ fixed_a, float fixed_dt) {
    constexpr int NP = NR * NS, PW = 64 / NS;
    extern __shared__ __align__(16) float lds[];
    float* sB = lds;                                   // [SSM_TB][NP]
    float* sC = sB + SSM_TB * NP;                      // [SSM_TB][NP]
    float* sX = sC + SSM_TB * NP;                      // [SSM_WAVES][SSM_TB][PW]
    float* sDt = sX + SSM_WAVES * SSM_TB * PW;         // [SSM_WAVES][SSM_TB]
    float* sA = sDt + SSM_WAVES * SSM_TB;              // [SSM_WAVES][SSM_TB]
    const int bx = blockIdx.x;
    const int seg = chunk_seg ? chunk_seg[bx] : bx;
    if (seg < 0) return;
    const int c = chunk_seg ? chunk_idx[bx] : 0;
    const int L = q_len[seg], first = c * Q;
    if (first >= L) return;
    const int ntok = (L - first < Q) ? L - first : Q;
    const bool last = first + ntok >= L;
    if (MODE == 1 && last) return;                      // nobody needs the last chunk's own state
    const int t0 = q_start[seg] + first;
    const int hpg = heads / G, PS = (vdim + PW - 1) / PW, U = hpg * PS, ublocks = (U + SSM_WAVES - 1) / SSM_WAVES;
    const int g = blockIdx.y / ublocks, ub = blockIdx.y % ublocks;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int unit = ub * SSM_WAVES + w;
    const bool active = unit < U;
    const int head = g * hpg + (active ? unit / PS : 0), pbase = active ? (unit % PS) * PW : 0;
    const int pl = lane / NS, s = lane % NS, p = pbase + pl;
    const int inner = heads * vdim;
    const size_t hoff = (size_t)head * N * vdim;
    float S[NR];
    if (MODE == 0 && active) {
        const float* src = chunk_seg ? carry + (size_t)bx * heads * N * vdim + hoff
                                     : state + (size_t)slots[seg] * heads * N * vdim + hoff;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int n = s * NR + r;
            S[r] = (n < N && p < vdim) ? src[(size_t)n * vdim + p] : 0.f;
        }
    } else {
#pragma unroll
        for (int r = 0; r < NR; ++r) S[r] = 0.f;
    }
    float prod = 1.f;
    const float Dh = (MODE == 0 && active && Dw) ? Dw[head] : 0.f;
    for (int b0 = 0; b0 < ntok; b0 += SSM_TB) {
        __syncthreads();
        for (int i = threadIdx.x; i < SSM_TB * NP; i += 64 * SSM_WAVES) {
            const int tt = i / NP, n = i % NP;
            const bool ok = b0 + tt < ntok && n < N;
            const float* row = xbc + (size_t)(t0 + b0 + tt) * xbc_stride + inner + (size_t)g * N + n;
            sB[i] = ok ? row[0] : 0.f;
            sC[i] = ok ? row[(size_t)G * N] : 0.f;
        }
        if (active) {
            for (int i = lane; i < SSM_TB * PW; i += 64) {
                const int tt = i / PW, pp = pbase + i % PW;
                const bool ok = b0 + tt < ntok && pp < vdim;
                sX[(w * SSM_TB + tt) * PW + i % PW] = ok ? xbc[(size_t)(t0 + b0 + tt) * xbc_stride + (size_t)head * vdim + pp] : 0.f;
            }
            if (lane < SSM_TB) {
                const bool ok = b0 + lane < ntok;
                // (a retention: the same decay and the same step for every token)
                const float d = !ok ? 0.f : fixed_a ? fixed_dt : softplus_f32(dt_raw[(size_t)(t0 + b0 + lane) * dt_stride + head] + dt_bias[head]);
                sDt[w * SSM_TB + lane] = d;
                sA[w * SSM_TB + lane] = fixed_a ? fixed_a[head] : expf(-expf(A_log[head]) * d);
            }
        }
        __syncthreads();
        if (!active) continue;
        const int nt = (ntok - b0 < SSM_TB) ? ntok - b0 : SSM_TB;
        for (int tt = 0; tt < nt; ++tt) {
            const float a = sA[w * SSM_TB + tt], dtv = sDt[w * SSM_TB + tt];
            const float xv = sX[(w * SSM_TB + tt) * PW + pl];
            const float dx = dtv * xv;
            const float4* Bp = reinterpret_cast<const float4*>(sB + tt * NP + s * NR);
            const float4* Cp = reinterpret_cast<const float4*>(sC + tt * NP + s * NR);
            float y0 = 0.f, y1 = 0.f, y2 = 0.f, y3 = 0.f;
#pragma unroll
            for (int r4 = 0; r4 < NR / 4; ++r4) {
                const float4 bv = Bp[r4];
                S[4 * r4 + 0] = fmaf(a, S[4 * r4 + 0], bv.x * dx);
                S[4 * r4 + 1] = fmaf(a, S[4 * r4 + 1], bv.y * dx);
                S[4 * r4 + 2] = fmaf(a, S[4 * r4 + 2], bv.z * dx);
                S[4 * r4 + 3] = fmaf(a, S[4 * r4 + 3], bv.w * dx);
                if (MODE == 0) {
                    const float4 cv = Cp[r4];
                    y0 = fmaf(S[4 * r4 + 0], cv.x, y0);
                    y1 = fmaf(S[4 * r4 + 1], cv.y, y1);
                    y2 = fmaf(S[4 * r4 + 2], cv.z, y2);
                    y3 = fmaf(S[4 * r4 + 3], cv.w, y3);
                }
            }
            if (MODE == 0) {
                float yv = (y0 + y1) + (y2 + y3);
#pragma unroll
                for (int o = 1; o < NS; o <<= 1) yv += __shfl_xor(yv, o, LI_WAVE);
                if (s == 0 && p < vdim) y[(size_t)(t0 + b0 + tt) * y_stride + (size_t)head * vdim + p] = fmaf(Dh, xv, yv);
            } else {
                prod *= a;
            }
        }
    }
    if (!active) return;
    float* dst = nullptr;
    if (MODE == 1) {
        dst = carry + (size_t)bx * heads * N * vdim + hoff;
        if (lane == 0 && pbase == 0) decay[(size_t)bx * heads + head] = prod;
    } else if (last) {
        dst = state + (size_t)slots[seg] * heads * N * vdim + hoff;
    }
    if (dst) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int n = s * NR + r;
            if (n < N && p < vdim) dst[(size_t)n * vdim + p] = S[r];
        }
    }
}

// The same recurrence with FOUR neighbouring columns a lane (head sizes that are multiples of 4): lane = quad * NS +
// slice holds NR state values of each of its four columns.  A value of B_t or C_t read from LDS then serves four
// state elements instead of one, and the state comes from and goes to memory in 16-byte pieces.  A wave is 256 / NS
// columns of one head.  Modes, chunks and blocks as above.
template <int NR, int NS, int MODE>
__global__ __launch_bounds__(64 * SSM_WAVES) void ssm_scan_quad_kernel(
    const float* __restrict__ xbc, long xbc_stride, const float* __restrict__ dt_raw, long dt_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dw,
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ q_start, const int* __restrict__ q_len,
    const int* __restrict__ chunk_seg, const int* __restrict__ chunk_idx, float* __restrict__ carry, float* __restrict__ decay,
    float* __restrict__ y, long y_stride, int heads, int vdim, int N, int G, int Q, const float* __restrict__ fixed_a, float fixed_dt) {
    constexpr int NP = NR * NS, PW = 256 / NS;
    extern __shared__ __align__(16) float lds[];
    float* sB = lds;                                   // [SSM_TB][NP]
    float* sC = sB + SSM_TB * NP;                      // [SSM_TB][NP]
    float* sX = sC + SSM_TB * NP;                      // [SSM_WAVES][SSM_TB][PW]
    float* sDt = sX + SSM_WAVES * SSM_TB * PW;         // [SSM_WAVES][SSM_TB]
    float* sA = sDt + SSM_WAVES * SSM_TB;              // [SSM_WAVES][SSM_TB]
    const int bx = blockIdx.x;
    const int seg = chunk_seg ? chunk_seg[bx] : bx;
    if (seg < 0) return;
    const int c = chunk_seg ? chunk_idx[bx] : 0;
    const int L = q_len[seg], first = c * Q;
    if (first >= L) return;
    const int ntok = (L - first < Q) ? L - first : Q;
    const bool last = first + ntok >= L;
    if (MODE == 1 && last) return;
    const int t0 = q_start[seg] + first;
    const int hpg = heads / G, PS = (vdim + PW - 1) / PW, U = hpg * PS, ublocks = (U + SSM_WAVES - 1) / SSM_WAVES;
    const int g = blockIdx.y / ublocks, ub = blockIdx.y % ublocks;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int unit = ub * SSM_WAVES + w;
    const bool active = unit < U;
    const int head = g * hpg + (active ? unit / PS : 0), pbase = active ? (unit % PS) * PW : 0;
    const int pq = lane / NS, s = lane % NS, p = pbase + 4 * pq;        // the first of the lane's four columns
    const bool cols = p < vdim;                                         // (vdim is a multiple of 4: all four or none)
    const int inner = heads * vdim;
    const size_t hoff = (size_t)head * N * vdim;
    float4 S[NR];
    if (MODE == 0 && active) {
        const float* src = chunk_seg ? carry + (size_t)bx * heads * N * vdim + hoff
                                     : state + (size_t)slots[seg] * heads * N * vdim + hoff;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int n = s * NR + r;
            S[r] = (n < N && cols) ? *reinterpret_cast<const float4*>(src + (size_t)n * vdim + p) : float4{0.f, 0.f, 0.f, 0.f};
        }
    } else {
#pragma unroll
        for (int r = 0; r < NR; ++r) S[r] = float4{0.f, 0.f, 0.f, 0.f};
    }
    float prod = 1.f;
    const float Dh = (MODE == 0 && active && Dw) ? Dw[head] : 0.f;
    for (int b0 = 0; b0 < ntok; b0 += SSM_TB) {
        __syncthreads();
        for (int i = threadIdx.x; i < SSM_TB * NP; i += 64 * SSM_WAVES) {
            const int tt = i / NP, n = i % NP;
            const bool ok = b0 + tt < ntok && n < N;
            const float* row = xbc + (size_t)(t0 + b0 + tt) * xbc_stride + inner + (size_t)g * N + n;
            sB[i] = ok ? row[0] : 0.f;
            sC[i] = ok ? row[(size_t)G * N] : 0.f;
        }
        if (active) {
            for (int i = lane; i < SSM_TB * PW; i += 64) {
                const int tt = i / PW, pp = pbase + i % PW;
                const bool ok = b0 + tt < ntok && pp < vdim;
                sX[(w * SSM_TB + tt) * PW + i % PW] = ok ? xbc[(size_t)(t0 + b0 + tt) * xbc_stride + (size_t)head * vdim + pp] : 0.f;
            }
            if (lane < SSM_TB) {
                const bool ok = b0 + lane < ntok;
                // (a retention: the same decay and the same step for every token)
                const float d = !ok ? 0.f : fixed_a ? fixed_dt : softplus_f32(dt_raw[(size_t)(t0 + b0 + lane) * dt_stride + head] + dt_bias[head]);
                sDt[w * SSM_TB + lane] = d;
                sA[w * SSM_TB + lane] = fixed_a ? fixed_a[head] : expf(-expf(A_log[head]) * d);
            }
        }
        __syncthreads();
        if (!active) continue;
        const int nt = (ntok - b0 < SSM_TB) ? ntok - b0 : SSM_TB;
        for (int tt = 0; tt < nt; ++tt) {
            const float a = sA[w * SSM_TB + tt], dtv = sDt[w * SSM_TB + tt];
            const float4 xv = *reinterpret_cast<const float4*>(sX + (w * SSM_TB + tt) * PW + 4 * pq);
            const float4 dx = float4{dtv * xv.x, dtv * xv.y, dtv * xv.z, dtv * xv.w};
            const float4* Bp = reinterpret_cast<const float4*>(sB + tt * NP + s * NR);
            const float4* Cp = reinterpret_cast<const float4*>(sC + tt * NP + s * NR);
            float4 yv = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int r4 = 0; r4 < NR / 4; ++r4) {
                const float4 bv = Bp[r4];
                const float bs[4] = {bv.x, bv.y, bv.z, bv.w};
                float cs[4] = {0.f, 0.f, 0.f, 0.f};
                if (MODE == 0) { const float4 cv = Cp[r4]; cs[0] = cv.x; cs[1] = cv.y; cs[2] = cv.z; cs[3] = cv.w; }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float4& st = S[4 * r4 + j];
                    st.x = fmaf(a, st.x, bs[j] * dx.x);
                    st.y = fmaf(a, st.y, bs[j] * dx.y);
                    st.z = fmaf(a, st.z, bs[j] * dx.z);
                    st.w = fmaf(a, st.w, bs[j] * dx.w);
                    if (MODE == 0) {
                        yv.x = fmaf(st.x, cs[j], yv.x);
                        yv.y = fmaf(st.y, cs[j], yv.y);
                        yv.z = fmaf(st.z, cs[j], yv.z);
                        yv.w = fmaf(st.w, cs[j], yv.w);
                    }
                }
            }
            if (MODE == 0) {
#pragma unroll
                for (int o = 1; o < NS; o <<= 1) {
                    yv.x += __shfl_xor(yv.x, o, LI_WAVE);
                    yv.y += __shfl_xor(yv.y, o, LI_WAVE);
                    yv.z += __shfl_xor(yv.z, o, LI_WAVE);
                    yv.w += __shfl_xor(yv.w, o, LI_WAVE);
                }
                if (s == 0 && cols)
                    *reinterpret_cast<float4*>(y + (size_t)(t0 + b0 + tt) * y_stride + (size_t)head * vdim + p) =
                        float4{fmaf(Dh, xv.x, yv.x), fmaf(Dh, xv.y, yv.y), fmaf(Dh, xv.z, yv.z), fmaf(Dh, xv.w, yv.w)};
            } else {
                prod *= a;
            }
        }
    }
    if (!active) return;
    float* dst = nullptr;
    if (MODE == 1) {
        dst = carry + (size_t)bx * heads * N * vdim + hoff;
        if (lane == 0 && pbase == 0) decay[(size_t)bx * heads + head] = prod;
    } else if (last) {
        dst = state + (size_t)slots[seg] * heads * N * vdim + hoff;
    }
    if (dst && cols) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int n = s * NR + r;
            if (n < N) *reinterpret_cast<float4*>(dst + (size_t)n * vdim + p) = S[r];
        }
    }
}

// Numbers the chunks of a step: request after request, chunk after chunk.  chunk_first[seg] is a request's
// first chunk; chunk_seg / chunk_idx say whose chunk, and which of its chunks, a number is (-1: none).
__global__ __launch_bounds__(256) void ssm_chunk_index_kernel(const int* __restrict__ q_len, int segs, int Q, int max_chunks,
                                                              int* __restrict__ chunk_seg, int* __restrict__ chunk_idx,
                                                              int* __restrict__ chunk_first) {
    if (threadIdx.x == 0) {
        int at = 0;
        for (int sgm = 0; sgm < segs; ++sgm) {
            chunk_first[sgm] = at;
            at += (q_len[sgm] + Q - 1) / Q;
        }
        chunk_first[segs] = at;
    }
    for (int i = threadIdx.x; i < max_chunks; i += 256) chunk_seg[i] = -1;
    __syncthreads();
    for (int sgm = threadIdx.x; sgm < segs; sgm += 256) {
        const int f = chunk_first[sgm], n = chunk_first[sgm + 1] - f;
        for (int k = 0; k < n && f + k < max_chunks; ++k) { chunk_seg[f + k] = sgm; chunk_idx[f + k] = k; }
    }
}

// carry[chunk] holds what the chunk alone built up from zero; afterwards it holds the state with which the
// chunk begins: the request's state for its first chunk, decay * (state before) + (built up before) onwards.
__global__ __launch_bounds__(256) void ssm_carry_kernel(float* __restrict__ carry, const float* __restrict__ decay,
                                                        const float* __restrict__ state, const int* __restrict__ slots,
                                                        const int* __restrict__ q_len, const int* __restrict__ chunk_first,
                                                        int heads, int NV, int Q) {
    const int seg = blockIdx.x, head = blockIdx.y;
    const int nch = (q_len[seg] + Q - 1) / Q, base = chunk_first[seg];
    const float* st = state + ((size_t)slots[seg] * heads + head) * NV;
    for (int e = blockIdx.z * 256 + threadIdx.x; e < NV; e += gridDim.z * 256) {
        float run = st[e];
        for (int k = 0; k < nch; ++k) {
            float* at = carry + ((size_t)(base + k) * heads + head) * NV + e;
            float next = 0.f;
            if (k + 1 < nch) next = fmaf(decay[(size_t)(base + k) * heads + head], run, *at);
            *at = run;
            run = next;
        }
    }
}

template <int NR, int NS, bool QUAD>
static int ssm_launch(const float* xbc, long xbc_stride, const float* dt_raw, long dt_stride, const float* dt_bias,
                      const float* A_log, const float* Dw, float* state, const int* slots, const int* q_start, const int* q_len,
                      int* chunk_tab, float* carry, float* decay, float* y, long y_stride, int heads, int vdim, int N, int G,
                      int Q, int segs, int max_chunks, bool chunked, const float* fixed_a, float fixed_dt, hipStream_t stream) {
    constexpr int NP = NR * NS, PW = (QUAD ? 256 : 64) / NS;
    const size_t lds = (size_t)(2 * SSM_TB * NP + SSM_WAVES * SSM_TB * PW + 2 * SSM_WAVES * SSM_TB) * sizeof(float);
#define SSM_KERNEL(MODE_) (QUAD ? ssm_scan_quad_kernel<(QUAD ? NR : 4), (QUAD ? NS : 2), MODE_> : ssm_scan_kernel<(QUAD ? 16 : NR), (QUAD ? 1 : NS), MODE_>)
    const int hpg = heads / G, PS = (vdim + PW - 1) / PW, U = hpg * PS, ublocks = (U + SSM_WAVES - 1) / SSM_WAVES;
    if (!chunked) {
        const dim3 grid(segs, G * ublocks);
        SSM_KERNEL(0)<<<grid, 64 * SSM_WAVES, lds, stream>>>(xbc, xbc_stride, dt_raw, dt_stride, dt_bias, A_log, Dw,
            state, slots, q_start, q_len, nullptr, nullptr, nullptr, nullptr, y, y_stride, heads, vdim, N, G, Q, fixed_a, fixed_dt);
        return li_launch_status();
    }
    int* chunk_seg = chunk_tab;
    int* chunk_idx = chunk_tab + max_chunks;
    int* chunk_first = chunk_tab + 2 * max_chunks;
    ssm_chunk_index_kernel<<<1, 256, 0, stream>>>(q_len, segs, Q, max_chunks, chunk_seg, chunk_idx, chunk_first);
    const dim3 grid(max_chunks, G * ublocks);
    SSM_KERNEL(1)<<<grid, 64 * SSM_WAVES, lds, stream>>>(xbc, xbc_stride, dt_raw, dt_stride, dt_bias, A_log, Dw,
        state, slots, q_start, q_len, chunk_seg, chunk_idx, carry, decay, y, y_stride, heads, vdim, N, G, Q, fixed_a, fixed_dt);
    const int NV = N * vdim;
    int zs = (NV + 255) / 256;
    if (zs > 16) zs = 16;
    ssm_carry_kernel<<<dim3(segs, heads, zs), 256, 0, stream>>>(carry, decay, state, slots, q_len, chunk_first, heads, NV, Q);
    SSM_KERNEL(0)<<<grid, 64 * SSM_WAVES, lds, stream>>>(xbc, xbc_stride, dt_raw, dt_stride, dt_bias, A_log, Dw,
        state, slots, q_start, q_len, chunk_seg, chunk_idx, carry, decay, y, y_stride, heads, vdim, N, G, Q, fixed_a, fixed_dt);
    return li_launch_status();
#undef SSM_KERNEL
}

// The four-columns-a-lane layout for a state of N values a column and heads of vdim columns (a multiple of 4): lanes
// a quad of columns (2 to 16) and values a lane and column (4 to 32); 0 if it has none.
static int ssm_quad_layout(int N, int vdim, int* slices, int* per_lane) {
    if (N <= 0 || N > 256 || vdim <= 0 || vdim % 4) return 0;
    int ns = 2;
    while (ns < 16 && 256 / (2 * ns) >= vdim) ns *= 2;      // narrow heads: more lanes a quad, so that a wave is full
    while (ns < 16 && (N + ns - 1) / ns > 32) ns *= 2;      // at most 32 values a lane and column (128 registers)
    const int need = (N + ns - 1) / ns;
    const int nr = need <= 4 ? 4 : need <= 8 ? 8 : need <= 16 ? 16 : need <= 32 ? 32 : 0;
    if (!nr || ns * nr > 256) return 0;
    *slices = ns;
    *per_lane = nr;
    return 1;
}

// How a state of N values a column is spread: slices (lanes a column) and values a lane; 0 if no kernel has it.
extern "C" int li_ssm_scan_layout(int N, int vdim, int* slices, int* per_lane) {
    if (N <= 0 || N > 256 || vdim <= 0) return 0;
    int ns = 1;
    while (ns < 4 && 64 / (2 * ns) >= vdim) ns *= 2;        // few columns a head: more lanes a column, so that a wave is full
    while (ns < 4 && (N + ns - 1) / ns > 128) ns *= 2;
    const int need = (N + ns - 1) / ns;
    int nr = need <= 16 ? 16 : need <= 32 ? 32 : need <= 64 ? 64 : need <= 128 ? 128 : 0;
    if (!nr) return 0;
    while (ns * nr > 256 && ns > 1 && (N + ns / 2 - 1) / (ns / 2) <= 128) {     // no more padding than LDS has room for
        ns /= 2;
        const int nd = (N + ns - 1) / ns;
        nr = nd <= 16 ? 16 : nd <= 32 ? 32 : nd <= 64 ? 64 : 128;
    }
    if (ns * nr > 256) return 0;
    if (slices) *slices = ns;
    if (per_lane) *per_lane = nr;
    return 1;
}

// Chunks that a step of T tokens in `segs` portions can have at most, and the bytes of the tables and states
// that the chunked form keeps in the workspace.
extern "C" long li_ssm_scan_work_bytes(int T, int segs, int heads, int vdim, int N, int Q, int* max_chunks) {
    const long mc = (long)T / Q + segs;
    if (max_chunks) *max_chunks = (int)mc;
    const long ints = ((3 * mc + segs + 1 + 3) / 4) * 4;
    return ints * 4 + mc * heads * ((long)N * vdim + 1) * 4;
}

extern "C" int li_ssm_scan(const float* xbc, long xbc_stride, const float* dt_raw, long dt_stride, const float* dt_bias,
                           const float* A_log, const float* Dw, float* state, const int* slots, const int* q_start,
                           const int* q_len, float* y, long y_stride, int heads, int vdim, int N, int G, int Q, int T,
                           int segs, int max_q_len, void* work, long work_bytes, const float* fixed_a, float fixed_dt, hipStream_t stream) {
    if (T <= 0 || segs <= 0 || heads <= 0 || G <= 0 || heads % G || vdim <= 0 || N <= 0 || Q <= 0 || max_q_len <= 0 ||
        xbc_stride < (long)heads * vdim + 2L * G * N || (!fixed_a && (dt_stride < heads || !dt_raw || !dt_bias || !A_log)) || y_stride < (long)heads * vdim)
        return LI_ERR_SIZE;
    int ns = 0, nr = 0;
    if (!li_ssm_scan_layout(N, vdim, &ns, &nr)) return LI_ERR_SIZE;
    const bool chunked = max_q_len > Q;
    int max_chunks = 0;
    int* chunk_tab = nullptr;
    float *carry = nullptr, *decay = nullptr;
    if (chunked) {
        const long need = li_ssm_scan_work_bytes(T, segs, heads, vdim, N, Q, &max_chunks);
        if (!work || work_bytes < need || ((uintptr_t)work % 16)) return LI_ERR_SIZE;
        chunk_tab = (int*)work;
        const long ints = ((3L * max_chunks + segs + 1 + 3) / 4) * 4;
        carry = (float*)work + ints;
        decay = carry + (size_t)max_chunks * heads * N * vdim;
    }
    const bool aligned = ((uintptr_t)state | (uintptr_t)y | (uintptr_t)carry) % 16 == 0 && y_stride % 4 == 0;
    int qs = 0, qr = 0;
    if (aligned && ssm_quad_layout(N, vdim, &qs, &qr)) {
#define SSM_QUAD(NR_, NS_)                                                                                                \
    if (qr == NR_ && qs == NS_)                                                                                           \
        return ssm_launch<NR_, NS_, true>(xbc, xbc_stride, dt_raw, dt_stride, dt_bias, A_log, Dw, state, slots, q_start, q_len, \
                                          chunk_tab, carry, decay, y, y_stride, heads, vdim, N, G, Q, segs, max_chunks, chunked, fixed_a, fixed_dt, stream);
        SSM_QUAD(4, 2) SSM_QUAD(8, 2) SSM_QUAD(16, 2) SSM_QUAD(32, 2)
        SSM_QUAD(4, 4) SSM_QUAD(8, 4) SSM_QUAD(16, 4) SSM_QUAD(32, 4)
        SSM_QUAD(4, 8) SSM_QUAD(8, 8) SSM_QUAD(16, 8) SSM_QUAD(32, 8)
        SSM_QUAD(4, 16) SSM_QUAD(8, 16) SSM_QUAD(16, 16) SSM_QUAD(32, 16)
#undef SSM_QUAD
    }
#define SSM_GO(NR_, NS_)                                                                                                  \
    if (nr == NR_ && ns == NS_)                                                                                           \
        return ssm_launch<NR_, NS_, false>(xbc, xbc_stride, dt_raw, dt_stride, dt_bias, A_log, Dw, state, slots, q_start, q_len,    \
                                    chunk_tab, carry, decay, y, y_stride, heads, vdim, N, G, Q, segs, max_chunks, chunked, fixed_a, fixed_dt, stream);
    SSM_GO(16, 1) SSM_GO(32, 1) SSM_GO(64, 1) SSM_GO(128, 1)
    SSM_GO(16, 2) SSM_GO(32, 2) SSM_GO(64, 2) SSM_GO(128, 2)
    SSM_GO(16, 4) SSM_GO(32, 4) SSM_GO(64, 4)
#undef SSM_GO
    return LI_ERR_SIZE;
}

// ------------------------------------------------------------------------------------ gated delta rule
// Per head, with a state S of N x vdim values:  S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;
// o_t = S^T q_t (the read-out sees the token's own write).  k_t and q_t are made unit vectors here
// (x / sqrt(sum x^2 + 1e-6)), q_t times q_scale; beta_t = sigmoid(b_t); g_t = exp(-exp(A_log) softplus(a_t + dt_bias)).
// Groups of heads share k and q.  A column of the state evolves by itself given the token's k, q, g, beta and its
// own v, so the layout is the state-space recurrence's: a lane owns CW neighbouring columns x NR state values,
// the NS slices of a column are neighbouring lanes that add up their shares of S^T k and of S^T q, a wave is
// 64 CW / NS columns of one head, the four waves of a block belong to ONE group and share k_t and q_t, which lie
// in LDS DR_TB tokens at a time (normed there: sixteen lanes a token add the squares in a fixed order).
// Rows of xkq: [v: heads x vdim | k: G x N | q: G x N]; rows of ba: [b: heads | a: heads].
#define DR_TB 16
//
// A step's portion of a request is cut into chunks of Q tokens that run side by side, as the state-space recurrence's
// are.  Here a token's step is S <- A_t S + beta_t k_t v_t^T with the MATRIX A_t = g_t (I - beta_t k_t k_t^T), so what a
// chunk does to the state it starts from is a matrix P = A_last ... A_first beside the state S_own that the chunk alone
// builds up from zero:
//   MODE 1: S_own of every chunk but a request's last, and P: its column j is what the recurrence, fed v = 0, makes of
//           the unit vector e_j, so P is N more columns of the same kernel (stored transposed: PT[j][n]);
//   the carry kernel: the state with which every chunk begins, chunk after chunk: S_in(c + 1) = P_c S_in(c) + S_own(c);
//   MODE 0: the recurrence itself from that state, with the outputs; the last chunk leaves the request's state.
// A portion of at most Q tokens (a decoding step) is MODE 0 alone, from the request's state.

template <int NR, int NS, int CW, int MODE>
__global__ __launch_bounds__(64 * SSM_WAVES) void delta_scan_kernel(
    const float* __restrict__ xkq, long x_stride, const float* __restrict__ ba, long ba_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ q_start, const int* __restrict__ q_len,
    const int* __restrict__ chunk_seg, const int* __restrict__ chunk_idx, float* __restrict__ carry, float* __restrict__ pmat,
    float* __restrict__ y, long y_stride, int heads, int vdim, int N, int G, int Q, float q_scale) {
    constexpr int NP = NR * NS, PW = 64 * CW / NS;
    extern __shared__ __align__(16) float lds[];
    float* sK = lds;                                   // [DR_TB][NP]
    float* sQ = sK + DR_TB * NP;                       // [DR_TB][NP]
    float* sX = sQ + DR_TB * NP;                       // [SSM_WAVES][DR_TB][PW]
    float* sBeta = sX + SSM_WAVES * DR_TB * PW;        // [SSM_WAVES][DR_TB]
    float* sG = sBeta + SSM_WAVES * DR_TB;             // [SSM_WAVES][DR_TB]
    const int bx = blockIdx.x;
    const int seg = chunk_seg ? chunk_seg[bx] : bx;
    if (seg < 0) return;
    const int c = chunk_seg ? chunk_idx[bx] : 0;
    const int L = q_len[seg], first = c * Q;
    if (first >= L) return;
    const int ntok = chunk_seg ? ((L - first < Q) ? L - first : Q) : L;
    const bool last = first + ntok >= L;
    if (MODE == 1 && last) return;                      // nobody needs the last chunk's own state
    const int t0 = q_start[seg] + first;
    // units of a head: blocks of PW value columns, and in MODE 1 behind them blocks of PW columns of P
    const int hpg = heads / G, PSV = (vdim + PW - 1) / PW, PS = PSV + (MODE == 1 ? (N + PW - 1) / PW : 0);
    const int U = hpg * PS, ublocks = (U + SSM_WAVES - 1) / SSM_WAVES;
    const int g = blockIdx.y / ublocks, ub = blockIdx.y % ublocks;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int unit = ub * SSM_WAVES + w;
    const bool active = unit < U;
    const int head = g * hpg + (active ? unit / PS : 0), sub = active ? unit % PS : 0;
    const bool is_p = MODE == 1 && sub >= PSV;
    const int pbase = (is_p ? sub - PSV : sub) * PW, ncols = is_p ? N : vdim;
    const int pq = lane / NS, s = lane % NS, p = pbase + CW * pq;       // the first of the lane's columns
    const int inner = heads * vdim;
    float* st = state + ((size_t)slots[seg] * heads + head) * N * vdim;
    const float* src = chunk_seg ? carry + ((size_t)bx * heads + head) * N * vdim : st;
    float S[NR][CW];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int n = s * NR + r;
        if (MODE == 1) {
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) S[r][cc] = (is_p && n == p + cc) ? 1.f : 0.f;
        } else if constexpr (CW == 4) {
            const float4 v4 = (active && n < N && p < vdim) ? *reinterpret_cast<const float4*>(src + (size_t)n * vdim + p)
                                                            : float4{0.f, 0.f, 0.f, 0.f};
            S[r][0] = v4.x; S[r][1] = v4.y; S[r][2] = v4.z; S[r][3] = v4.w;
        } else {
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) S[r][cc] = (active && n < N && p + cc < vdim) ? src[(size_t)n * vdim + p + cc] : 0.f;
        }
    }
    for (int b0 = 0; b0 < ntok; b0 += DR_TB) {
        __syncthreads();
        for (int i = threadIdx.x; i < DR_TB * NP; i += 64 * SSM_WAVES) {
            const int tt = i / NP, n = i % NP;
            const bool ok = b0 + tt < ntok && n < N;
            const float* row = xkq + (size_t)(t0 + b0 + tt) * x_stride + inner + (size_t)g * N + n;
            sK[i] = ok ? row[0] : 0.f;
            sQ[i] = ok ? row[(size_t)G * N] : 0.f;
        }
        if (active) {
            for (int i = lane; i < DR_TB * PW; i += 64) {
                const int tt = i / PW, pp = pbase + i % PW;
                const bool ok = !is_p && b0 + tt < ntok && pp < vdim;
                sX[(w * DR_TB + tt) * PW + i % PW] = ok ? xkq[(size_t)(t0 + b0 + tt) * x_stride + (size_t)head * vdim + pp] : 0.f;
            }
            if (lane < DR_TB) {
                const bool ok = b0 + lane < ntok;
                const float* r2 = ba + (size_t)(t0 + b0 + (ok ? lane : 0)) * ba_stride;
                sBeta[w * DR_TB + lane] = ok ? 1.0f / (1.0f + expf(-r2[head])) : 0.f;
                sG[w * DR_TB + lane] = ok ? expf(-expf(A_log[head]) * softplus_f32(r2[heads + head] + dt_bias[head])) : 1.f;
            }
        }
        __syncthreads();
        {   // unit vectors: token tt = thread / 16, sixteen neighbouring lanes share its N values
            const int tt = threadIdx.x >> 4, part = threadIdx.x & 15;
            float sk = 0.f, sq = 0.f;
            for (int n = part; n < NP; n += 16) {
                const float kv = sK[tt * NP + n], qv = sQ[tt * NP + n];
                sk = fmaf(kv, kv, sk);
                sq = fmaf(qv, qv, sq);
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) {
                sk += __shfl_xor(sk, o, LI_WAVE);
                sq += __shfl_xor(sq, o, LI_WAVE);
            }
            const float ik = 1.0f / sqrtf(sk + 1e-6f), iq = q_scale / sqrtf(sq + 1e-6f);
            for (int n = part; n < NP; n += 16) {
                sK[tt * NP + n] *= ik;
                sQ[tt * NP + n] *= iq;
            }
        }
        __syncthreads();
        if (!active) continue;
        const int nt = (ntok - b0 < DR_TB) ? ntok - b0 : DR_TB;
        for (int tt = 0; tt < nt; ++tt) {
            const float gd = sG[w * DR_TB + tt], beta = sBeta[w * DR_TB + tt];
            float xv[CW];
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) xv[cc] = sX[(w * DR_TB + tt) * PW + CW * pq + cc];
            const float4* Kp = reinterpret_cast<const float4*>(sK + tt * NP + s * NR);
            const float4* Qp = reinterpret_cast<const float4*>(sQ + tt * NP + s * NR);
            float ks[CW];
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) ks[cc] = 0.f;
#pragma unroll
            for (int r4 = 0; r4 < NR / 4; ++r4) {
                const float4 kv = Kp[r4];
                const float kk[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int cc = 0; cc < CW; ++cc) ks[cc] = fmaf(S[4 * r4 + j][cc], kk[j], ks[cc]);
            }
#pragma unroll
            for (int o = 1; o < NS; o <<= 1)
#pragma unroll
                for (int cc = 0; cc < CW; ++cc) ks[cc] += __shfl_xor(ks[cc], o, LI_WAVE);
            float u[CW], ov[CW];
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) { u[cc] = beta * (xv[cc] - gd * ks[cc]); ov[cc] = 0.f; }
#pragma unroll
            for (int r4 = 0; r4 < NR / 4; ++r4) {
                const float4 kv = Kp[r4];
                const float kk[4] = {kv.x, kv.y, kv.z, kv.w};
                float qs[4] = {0.f, 0.f, 0.f, 0.f};
                if (MODE == 0) { const float4 qv = Qp[r4]; qs[0] = qv.x; qs[1] = qv.y; qs[2] = qv.z; qs[3] = qv.w; }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int cc = 0; cc < CW; ++cc) {
                        const float nv = fmaf(gd, S[4 * r4 + j][cc], kk[j] * u[cc]);
                        S[4 * r4 + j][cc] = nv;
                        if (MODE == 0) ov[cc] = fmaf(nv, qs[j], ov[cc]);
                    }
            }
            if (MODE == 0) {
#pragma unroll
                for (int o = 1; o < NS; o <<= 1)
#pragma unroll
                    for (int cc = 0; cc < CW; ++cc) ov[cc] += __shfl_xor(ov[cc], o, LI_WAVE);
                if (s == 0) {
                    float* yr = y + (size_t)(t0 + b0 + tt) * y_stride + (size_t)head * vdim + p;
                    if constexpr (CW == 4) {
                        if (p < vdim) *reinterpret_cast<float4*>(yr) = float4{ov[0], ov[1], ov[2], ov[3]};
                    } else {
#pragma unroll
                        for (int cc = 0; cc < CW; ++cc) if (p + cc < vdim) yr[cc] = ov[cc];
                    }
                }
            }
        }
    }
    if (!active) return;
    if (MODE == 1 && is_p) {                            // PT[j][n]: the lane's columns j, its n values side by side
        float* pt = pmat + ((size_t)bx * heads + head) * N * N;
#pragma unroll
        for (int cc = 0; cc < CW; ++cc)
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                const int n = s * NR + r;
                if (n < N && p + cc < N) pt[(size_t)(p + cc) * N + n] = S[r][cc];
            }
        return;
    }
    float* dst = MODE == 1 ? carry + ((size_t)bx * heads + head) * N * vdim : (last ? st : nullptr);
    if (!dst) return;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int n = s * NR + r;
        if (n >= N) continue;
        if constexpr (CW == 4) {
            if (p < vdim) *reinterpret_cast<float4*>(dst + (size_t)n * vdim + p) = float4{S[r][0], S[r][1], S[r][2], S[r][3]};
        } else {
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) if (p + cc < vdim) dst[(size_t)n * vdim + p + cc] = S[r][cc];
        }
    }
    (void)ncols;
}

// carry[chunk] holds what the chunk alone built up from zero, pmat[chunk] its matrix (transposed); afterwards carry[chunk]
// holds the state with which the chunk begins.  A block takes a request, a head and DC_COLS columns of the state, chunk
// after chunk; the state's columns lie in LDS, thread (slice, column) owns PER consecutive values of the column
// (DC_SLICES * PER >= N).  A chunk's step is a product P x (state's columns): the thread walks P's rows j, which hold its
// PER values side by side, DC_AHEAD rows at a time: their loads are issued
// together and without conditions (a value past N reads the row's last one and is never stored), so that a trip to memory
// serves DC_AHEAD rows and not one.
#define DC_COLS 16
#define DC_SLICES 16
#define DC_ROUND 16                 // the state's rows in LDS are rounded up to this: the most rows a trip takes
template <int PER, int DC_AHEAD, bool VEC>      // VEC: N and PER multiples of 4, P on 16 bytes: a row's values in 16-byte pieces
__global__ __launch_bounds__(DC_COLS * DC_SLICES) void delta_carry_kernel(
    float* __restrict__ carry, const float* __restrict__ pmat, const float* __restrict__ state, const int* __restrict__ slots,
    const int* __restrict__ q_len, const int* __restrict__ chunk_first, int heads, int vdim, int N, int Q) {
    extern __shared__ float run[];                      // [N rounded up to DC_ROUND][DC_COLS + 1]
    const int seg = blockIdx.x, head = blockIdx.y, cl = threadIdx.x % DC_COLS, sl = threadIdx.x / DC_COLS;
    const int col = blockIdx.z * DC_COLS + cl;
    const int nch = (q_len[seg] + Q - 1) / Q, base = chunk_first[seg];
    const int n0 = sl * PER;
    const bool on = col < vdim;
    const int NA = (N + DC_ROUND - 1) / DC_ROUND * DC_ROUND;
    const float* stp = state + ((size_t)slots[seg] * heads + head) * N * vdim;
    int off[PER];                                       // the thread's values within a row of P (clamped: loads carry no conditions)
#pragma unroll
    for (int i = 0; i < PER; ++i) off[i] = n0 + i < N ? n0 + i : N - 1;
#pragma unroll
    for (int i = 0; i < PER; ++i)
        if (n0 + i < NA) run[(n0 + i) * (DC_COLS + 1) + cl] = (on && n0 + i < N) ? stp[(size_t)(n0 + i) * vdim + col] : 0.f;
    __syncthreads();
    for (int k = 0; k < nch; ++k) {
        float* at = carry + ((size_t)(base + k) * heads + head) * N * vdim;
        const float* pt = pmat + ((size_t)(base + k) * heads + head) * N * N;
        float acc[PER];
        const bool more = k + 1 < nch;
#pragma unroll
        for (int i = 0; i < PER; ++i) acc[i] = (more && on && n0 + i < N) ? at[(size_t)(n0 + i) * vdim + col] : 0.f;
        if (more) {
            for (int j0 = 0; j0 < N; j0 += DC_AHEAD) {
                float pv[DC_AHEAD][PER], cv[DC_AHEAD];
#pragma unroll
                for (int u = 0; u < DC_AHEAD; ++u) {
                    const float* prow = pt + (size_t)(j0 + u < N ? j0 + u : N - 1) * N;
                    if constexpr (VEC) {
#pragma unroll
                        for (int v = 0; v < PER / 4; ++v) {
                            const float4 t4 = *reinterpret_cast<const float4*>(prow + (n0 + 4 * v < N ? n0 + 4 * v : N - 4));
                            pv[u][4 * v] = t4.x; pv[u][4 * v + 1] = t4.y; pv[u][4 * v + 2] = t4.z; pv[u][4 * v + 3] = t4.w;
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < PER; ++i) pv[u][i] = prow[off[i]];
                    }
                    cv[u] = run[(j0 + u) * (DC_COLS + 1) + cl];             // (rows N .. NA - 1 of the state are zeros)
                }
#pragma unroll
                for (int u = 0; u < DC_AHEAD; ++u)
#pragma unroll
                    for (int i = 0; i < PER; ++i) acc[i] = fmaf(pv[u][i], cv[u], acc[i]);
            }
        }
        // the chunk begins with `run`; the next one with what has just been added up
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (on && n0 + i < N) at[(size_t)(n0 + i) * vdim + col] = run[(n0 + i) * (DC_COLS + 1) + cl];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (n0 + i < N) run[(n0 + i) * (DC_COLS + 1) + cl] = acc[i];
        __syncthreads();
    }
}

static void delta_carry_launch(float* carry, const float* pmat, const float* state, const int* slots, const int* q_len,
                               const int* chunk_first, int heads, int vdim, int N, int Q, int segs, hipStream_t stream) {
    const dim3 grid(segs, heads, (vdim + DC_COLS - 1) / DC_COLS);
    const size_t lds = (size_t)((N + DC_ROUND - 1) / DC_ROUND * DC_ROUND) * (DC_COLS + 1) * sizeof(float);
    const int per = (N + DC_SLICES - 1) / DC_SLICES;
#define DC_GO(P_, V_) delta_carry_kernel<P_, 8, V_><<<grid, DC_COLS * DC_SLICES, lds, stream>>>(carry, pmat, state, slots, q_len, chunk_first, heads, vdim, N, Q)
    const bool vec = N % 4 == 0 && ((uintptr_t)pmat % 16) == 0;
    if (per <= 1) DC_GO(1, false); else if (per <= 2) DC_GO(2, false);
    else if (per <= 4) { if (vec) DC_GO(4, true); else DC_GO(4, false); }
    else if (per <= 8) { if (vec) DC_GO(8, true); else DC_GO(8, false); }
    else { if (vec) DC_GO(16, true); else DC_GO(16, false); }
#undef DC_GO
}

template <int NR, int NS, int CW>
static int delta_launch(const float* xkq, long x_stride, const float* ba, long ba_stride, const float* dt_bias, const float* A_log,
                        float* state, const int* slots, const int* q_start, const int* q_len, int* chunk_tab, float* carry,
                        float* pmat, float* y, long y_stride, int heads, int vdim, int N, int G, int Q, float q_scale, int segs,
                        int max_chunks, bool chunked, hipStream_t stream) {
    constexpr int NP = NR * NS, PW = 64 * CW / NS;
    const size_t lds = (size_t)(2 * DR_TB * NP + SSM_WAVES * DR_TB * PW + 2 * SSM_WAVES * DR_TB) * sizeof(float);
    const int hpg = heads / G, PSV = (vdim + PW - 1) / PW, PSP = (N + PW - 1) / PW;
    const int ub0 = (hpg * PSV + SSM_WAVES - 1) / SSM_WAVES, ub1 = (hpg * (PSV + PSP) + SSM_WAVES - 1) / SSM_WAVES;
    if (!chunked) {
        delta_scan_kernel<NR, NS, CW, 0><<<dim3(segs, G * ub0), 64 * SSM_WAVES, lds, stream>>>(
            xkq, x_stride, ba, ba_stride, dt_bias, A_log, state, slots, q_start, q_len, nullptr, nullptr, nullptr, nullptr,
            y, y_stride, heads, vdim, N, G, Q, q_scale);
        return li_launch_status();
    }
    int* chunk_seg = chunk_tab;
    int* chunk_idx = chunk_tab + max_chunks;
    int* chunk_first = chunk_tab + 2 * max_chunks;
    ssm_chunk_index_kernel<<<1, 256, 0, stream>>>(q_len, segs, Q, max_chunks, chunk_seg, chunk_idx, chunk_first);
    delta_scan_kernel<NR, NS, CW, 1><<<dim3(max_chunks, G * ub1), 64 * SSM_WAVES, lds, stream>>>(
        xkq, x_stride, ba, ba_stride, dt_bias, A_log, state, slots, q_start, q_len, chunk_seg, chunk_idx, carry, pmat,
        y, y_stride, heads, vdim, N, G, Q, q_scale);
    delta_carry_launch(carry, pmat, state, slots, q_len, chunk_first, heads, vdim, N, Q, segs, stream);
    delta_scan_kernel<NR, NS, CW, 0><<<dim3(max_chunks, G * ub0), 64 * SSM_WAVES, lds, stream>>>(
        xkq, x_stride, ba, ba_stride, dt_bias, A_log, state, slots, q_start, q_len, chunk_seg, chunk_idx, carry, pmat,
        y, y_stride, heads, vdim, N, G, Q, q_scale);
    return li_launch_status();
}

// 1 if the recurrence has a layout for a state of N values a column (the state-space recurrence's layouts)
extern "C" int li_delta_scan_takes(int N, int vdim) { return li_ssm_scan_layout(N, vdim, nullptr, nullptr); }

// Chunks that a step of T tokens in `segs` portions can have at most, and the bytes of the tables, states and matrices
// that the chunked form keeps in the workspace.
extern "C" long li_delta_scan_work_bytes(int T, int segs, int heads, int vdim, int N, int Q, int* max_chunks) {
    const long mc = (long)T / Q + segs;
    if (max_chunks) *max_chunks = (int)mc;
    const long ints = ((3 * mc + segs + 1 + 3) / 4) * 4;
    return ints * 4 + mc * heads * ((long)N * vdim + (long)N * N) * 4;
}

extern "C" int li_delta_scan(const float* xkq, long x_stride, const float* ba, long ba_stride, const float* dt_bias,
                             const float* A_log, float* state, const int* slots, const int* q_start, const int* q_len,
                             float* y, long y_stride, int heads, int vdim, int N, int G, float q_scale, int Q, int T, int segs,
                             int max_q_len, void* work, long work_bytes, hipStream_t stream) {
    if (T <= 0 || segs <= 0 || heads <= 0 || G <= 0 || heads % G || vdim <= 0 || N <= 0 || N > 256 || Q <= 0 || max_q_len <= 0 ||
        x_stride < (long)heads * vdim + 2L * G * N || ba_stride < 2L * heads || y_stride < (long)heads * vdim)
        return LI_ERR_SIZE;
    const bool chunked = max_q_len > Q;
    int max_chunks = 0;
    int* chunk_tab = nullptr;
    float *carry = nullptr, *pmat = nullptr;
    if (chunked) {
        const long need = li_delta_scan_work_bytes(T, segs, heads, vdim, N, Q, &max_chunks);
        if (!work || work_bytes < need || ((uintptr_t)work % 16)) return LI_ERR_SIZE;
        chunk_tab = (int*)work;
        const long ints = ((3L * max_chunks + segs + 1 + 3) / 4) * 4;
        carry = (float*)work + ints;
        pmat = carry + (size_t)max_chunks * heads * N * vdim;
    }
#define DR_ARGS xkq, x_stride, ba, ba_stride, dt_bias, A_log, state, slots, q_start, q_len, chunk_tab, carry, pmat, y, y_stride, heads, \
                vdim, N, G, Q, q_scale, segs, max_chunks, chunked, stream
    const bool aligned = ((uintptr_t)state | (uintptr_t)y | (uintptr_t)carry) % 16 == 0 && y_stride % 4 == 0;
    int qs = 0, qr = 0;
    if (aligned && ssm_quad_layout(N, vdim, &qs, &qr)) {
#define DR_QUAD(NR_, NS_) if (qr == NR_ && qs == NS_) return delta_launch<NR_, NS_, 4>(DR_ARGS);
        DR_QUAD(4, 2) DR_QUAD(8, 2) DR_QUAD(16, 2) DR_QUAD(32, 2)
        DR_QUAD(4, 4) DR_QUAD(8, 4) DR_QUAD(16, 4) DR_QUAD(32, 4)
        DR_QUAD(4, 8) DR_QUAD(8, 8) DR_QUAD(16, 8) DR_QUAD(32, 8)
        DR_QUAD(4, 16) DR_QUAD(8, 16) DR_QUAD(16, 16)
#undef DR_QUAD
    }
    int ns = 0, nr = 0;
    if (!li_ssm_scan_layout(N, vdim, &ns, &nr)) return LI_ERR_SIZE;
#define DR_GO(NR_, NS_) if (nr == NR_ && ns == NS_) return delta_launch<NR_, NS_, 1>(DR_ARGS);
    DR_GO(16, 1) DR_GO(32, 1) DR_GO(64, 1) DR_GO(128, 1)
    DR_GO(16, 2) DR_GO(32, 2) DR_GO(64, 2) DR_GO(128, 2)
    DR_GO(16, 4) DR_GO(32, 4) DR_GO(64, 4)
#undef DR_GO
#undef DR_ARGS
    return LI_ERR_SIZE;
}

// ------------------------------------------------------------------------------------ gated norm in groups
// Every group of `gs` neighbouring columns has its own root mean square.  gate_after 0: out[t, c] = w[c] * v /
// sqrt(mean of v^2 over c's group + eps) with v = y[t, c] * silu(z[t, c]): the gate comes before the norm.
// gate_after 1: out[t, c] = w[c] * y / sqrt(mean of y^2 + eps) * silu(z[t, c]): the norm sees y alone.  w null: ones.
// A block a (token, group).
template <typename TO, int PER>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, long y_stride,
                                                               const float* __restrict__ z, long z_stride,
                                                               const float* __restrict__ w, float eps, TO* __restrict__ out,
                                                               long out_stride, int gs, int gate_after) {
    __shared__ float red[256 / LI_WAVE];
    const int t = blockIdx.x, c0 = blockIdx.y * gs;
    const float* yr = y + (size_t)t * y_stride + c0;
    const float* zr = z + (size_t)t * z_stride + c0;
    float v[PER], gt[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * 256;
        float g = 0.f, sg = 0.f;
        if (j < gs) { const float zz = zr[j]; sg = zz / (1.0f + expf(-zz)); g = gate_after ? yr[j] : yr[j] * sg; }
        v[i] = g;
        gt[i] = gate_after ? sg : 1.f;
        ss += g * g;
    }
    for (int j = threadIdx.x + PER * 256; j < gs; j += 256) {
        const float zz = zr[j], sg = zz / (1.0f + expf(-zz)), g = gate_after ? yr[j] : yr[j] * sg;
        ss += g * g;
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    TO* o = out + (size_t)t * out_stride + c0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * 256;
        if (j < gs) store_from_float(o + j, (w ? w[c0 + j] : 1.f) * v[i] * inv * gt[i]);
    }
    for (int j = threadIdx.x + PER * 256; j < gs; j += 256) {
        const float zz = zr[j], sg = zz / (1.0f + expf(-zz)), g = gate_after ? yr[j] : yr[j] * sg;
        store_from_float(o + j, (w ? w[c0 + j] : 1.f) * g * inv * (gate_after ? sg : 1.f));
    }
}

extern "C" int li_gated_group_norm(const float* y, long y_stride, const float* z, long z_stride, const float* w, float eps,
                                   void* out, int out_dtype, long out_stride, int T, int n, int groups, int gate_after,
                                   hipStream_t stream) {
    if (T <= 0 || n <= 0 || groups <= 0 || n % groups || groups > 65535 || y_stride < n || z_stride < n || out_stride < n)
        return LI_ERR_SIZE;
    const dim3 grid(T, groups);
    if (out_dtype == LI_F32)
        gated_group_norm_kernel<float, 8><<<grid, 256, 0, stream>>>(y, y_stride, z, z_stride, w, eps, (float*)out, out_stride, n / groups, gate_after);
    else if (out_dtype == LI_BF16)
        gated_group_norm_kernel<bf16_t, 8><<<grid, 256, 0, stream>>>(y, y_stride, z, z_stride, w, eps, (bf16_t*)out, out_stride, n / groups, gate_after);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}
