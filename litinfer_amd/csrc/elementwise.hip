// Row-wise and element-wise kernels: embedding gather, RMSNorm, row gather,
// casts, SwiGLU, rotary tables and rotation, and the write of keys and values
// into their pages.  Arithmetic is float32 throughout; bfloat16 is a storage
// format that is widened on load and rounded once on store.
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[t, :] = float(table[id(t), :])  (row copy, no scaling), with id(t) = ids[t], or, where
// id_src is given and id_src[t] >= 0, feedback[id_src[t]]: a token that an earlier kernel on the
// stream chose and the host has not seen yet.
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const int* __restrict__ id_src,
                                 const int* __restrict__ feedback, const T* __restrict__ table,
                                 float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id_src) {
        const int src = id_src[t];
        if (src >= 0) id = feedback[src];
    }
    float* o = out + (size_t)t * H;
    if (id < 0 || id >= V) {                       // the host has checked what it knows; never read outside:
        for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = 0.f;      // a row of zeros, not what an earlier step left
        return;
    }
    const T* row = table + (size_t)id * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = load_as_float(row + j);
}

extern "C" int li_embedding(const int* ids, const int* id_src, const int* feedback, const void* table,
                            int table_dtype, float* out, int T, int H, int V, hipStream_t stream) {
    if (T <= 0 || H <= 0 || (id_src && !feedback)) return LI_ERR_SIZE;
    if (table_dtype == LI_F32)
        embedding_kernel<float><<<T, 256, 0, stream>>>(ids, id_src, feedback, (const float*)table, out, H, V);
    else if (table_dtype == LI_BF16)
        embedding_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, id_src, feedback, (const bf16_t*)table, out, H, V);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ------------------------------------------------------------------ rmsnorm
// y = w * x * rsqrt(mean(x^2) + eps), eps inside the root; one block per row.  The row is
// read once and kept in registers (up to RN_PER elements a thread); longer rows are read again.
// Few rows (a decoding step): 1024 threads a row, so that the one row is read with the least
// latency; many rows (a prompt): 256 threads a row, less of a block's time goes into meeting.
template <typename TI, typename TO, int NT, int PER>
__global__ __launch_bounds__(NT) void rmsnorm_kernel(const TI* __restrict__ x, const float* __restrict__ w,
                                                      float eps, TO* __restrict__ out, int H) {
    __shared__ float red[NT / LI_WAVE];
    const TI* row = x + (size_t)blockIdx.x * H;
    TO* o = out + (size_t)blockIdx.x * H;
    float v[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        v[i] = (j < H) ? load_as_float(row + j) : 0.f;
        ss += v[i] * v[i];
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT) { const float t = load_as_float(row + j); ss += t * t; }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        if (j < H) store_from_float(o + j, w[j] * v[i] * inv);
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT)
        store_from_float(o + j, w[j] * load_as_float(row + j) * inv);
}

// Many rows of float32 whose length is a multiple of 4 (a prompt's residual rows): 16 bytes a lane.
template <typename TO, int NT, int PER>
__global__ __launch_bounds__(NT) void rmsnorm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                          float eps, TO* __restrict__ out, int H) {
    __shared__ float red[NT / LI_WAVE];
    const float4* row = reinterpret_cast<const float4*>(x + (size_t)blockIdx.x * H);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    TO* o = out + (size_t)blockIdx.x * H;
    const int n4 = H / 4;
    float4 v[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        v[i] = (j < n4) ? row[j] : float4{0.f, 0.f, 0.f, 0.f};
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        if (j < n4) {
            const float4 g = w4[j];
            const float y0 = g.x * v[i].x * inv, y1 = g.y * v[i].y * inv, y2 = g.z * v[i].z * inv, y3 = g.w * v[i].w * inv;
            if constexpr (sizeof(TO) == 2) {
                *reinterpret_cast<uint2*>(o + 4 * j) = uint2{pack2_bf16(y0, y1), pack2_bf16(y2, y3)};
            } else {
                *reinterpret_cast<float4*>(o + 4 * j) = float4{y0, y1, y2, y3};
            }
        }
    }
}

extern "C" int li_rmsnorm(const void* x, int x_dtype, const float* w, float eps, void* out,
                          int out_dtype, int T, int H, hipStream_t stream) {
    if (T <= 0 || H <= 0) return LI_ERR_SIZE;
#define LI_NORM(TI, TO)                                                                                        \
    {                                                                                                          \
        if (T >= 256) rmsnorm_kernel<TI, TO, 256, 16><<<T, 256, 0, stream>>>((const TI*)x, w, eps, (TO*)out, H); \
        else rmsnorm_kernel<TI, TO, 1024, 8><<<T, 1024, 0, stream>>>((const TI*)x, w, eps, (TO*)out, H);        \
    }
    if (x_dtype == LI_F32 && T >= 256 && H % 4 == 0 && H <= 4 * 256 * 8 && ((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) % 16 == 0) {
        if (out_dtype == LI_F32) rmsnorm_vec_kernel<float, 256, 8><<<T, 256, 0, stream>>>((const float*)x, w, eps, (float*)out, H);
        else if (out_dtype == LI_BF16) rmsnorm_vec_kernel<bf16_t, 256, 8><<<T, 256, 0, stream>>>((const float*)x, w, eps, (bf16_t*)out, H);
        else return LI_ERR_DTYPE;
        return li_launch_status();
    }
    if (x_dtype == LI_F32 && out_dtype == LI_F32) LI_NORM(float, float)
    else if (x_dtype == LI_F32 && out_dtype == LI_BF16) LI_NORM(float, bf16_t)
    else if (x_dtype == LI_BF16 && out_dtype == LI_BF16) LI_NORM(bf16_t, bf16_t)
    else if (x_dtype == LI_BF16 && out_dtype == LI_F32) LI_NORM(bf16_t, float)
    else return LI_ERR_DTYPE;
#undef LI_NORM
    return li_launch_status();
}

// -------------------------------------------------------------- gather rows
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                   float* __restrict__ out, int H) {
    const float* src = x + (size_t)rows[blockIdx.x] * H;
    float* dst = out + (size_t)blockIdx.x * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = src[j];
}

extern "C" int li_gather_rows(const float* x, const int* rows, float* out, int n, int H,
                              hipStream_t stream) {
    if (n <= 0 || H <= 0) return LI_ERR_SIZE;
    gather_rows_kernel<<<n, 256, 0, stream>>>(x, rows, out, H);
    return li_launch_status();
}

// --------------------------------------------------------------------- cast
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ src, TO* __restrict__ dst, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        store_from_float(dst + i, load_as_float(src + i));
}

extern "C" int li_cast(const void* src, int sdt, void* dst, int ddt, long n, hipStream_t stream) {
    if (n <= 0) return LI_ERR_SIZE;
    long blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (sdt == LI_F32 && ddt == LI_BF16) cast_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((const float*)src, (bf16_t*)dst, n);
    else if (sdt == LI_BF16 && ddt == LI_F32) cast_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>((const bf16_t*)src, (float*)dst, n);
    else if (sdt == LI_F32 && ddt == LI_F32) cast_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)src, (float*)dst, n);
    else if (sdt == LI_BF16 && ddt == LI_BF16) cast_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)src, (bf16_t*)dst, n);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ------------------------------------------------------------------- swiglu
// out[t, i] = up * gate / (1 + exp(-gate)), gate = gu[t, i], up = gu[t, I + i]
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I) {
    const T* g = gu + (size_t)blockIdx.y * 2 * I;
    T* o = out + (size_t)blockIdx.y * I;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < I) {
        const float gv = load_as_float(g + i), uv = load_as_float(g + I + i);
        store_from_float(o + i, uv * (gv / (1.0f + expf(-gv))));
    }
}

extern "C" int li_swiglu(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream) {
    if (T <= 0 || I <= 0 || T > 65535 * 32) return LI_ERR_SIZE;
    // grid.y is limited to 65535: walk the rows in slabs
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int rows = (T - t0 < 65535) ? T - t0 : 65535;
        dim3 grid((I + 255) / 256, rows);
        if (dtype == LI_F32)
            swiglu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu + (size_t)t0 * 2 * I, (float*)out + (size_t)t0 * I, I);
        else if (dtype == LI_BF16)
            swiglu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I);
        else return LI_ERR_DTYPE;
    }
    return li_launch_status();
}

// out[t, i] = act(gate) * up with gate = gu[t, i], up = gu[t, I + i]; act 0: z / (1 + exp(-z)),
// act 1: the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))).  Arithmetic in float32.
template <typename TI, typename TO>
__global__ void gated_act_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int I, int act) {
    const TI* g = gu + (size_t)blockIdx.y * 2 * I;
    TO* o = out + (size_t)blockIdx.y * I;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < I) {
        const float gv = load_as_float(g + i), uv = load_as_float(g + I + i);
        const float a = act == 1 ? 0.5f * gv * (1.0f + tanhf(0.7978845608028654f * (gv + 0.044715f * gv * gv * gv)))
                                 : gv / (1.0f + expf(-gv));
        store_from_float(o + i, a * uv);
    }
}

extern "C" int li_gated_act(const void* gu, int in_dtype, void* out, int out_dtype, int T, int I, int act, hipStream_t stream) {
    if (T <= 0 || I <= 0 || T > 65535 * 32 || act < 0 || act > 1) return LI_ERR_SIZE;
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int rows = (T - t0 < 65535) ? T - t0 : 65535;
        dim3 grid((I + 255) / 256, rows);
        if (in_dtype == LI_F32 && out_dtype == LI_F32)
            gated_act_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)gu + (size_t)t0 * 2 * I, (float*)out + (size_t)t0 * I, I, act);
        else if (in_dtype == LI_F32 && out_dtype == LI_BF16)
            gated_act_kernel<float, bf16_t><<<grid, 256, 0, stream>>>((const float*)gu + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I, act);
        else if (in_dtype == LI_BF16 && out_dtype == LI_BF16)
            gated_act_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I, act);
        else return LI_ERR_DTYPE;
    }
    return li_launch_status();
}

// --------------------------------------------------------------------- rope
// angle = float(pos) / powf(theta, float(2j) / rotary_dim); cos and sin in float32
__global__ void rope_table_kernel(const int* __restrict__ pos, float theta, int rotary_dim,
                                  float* __restrict__ cosv, float* __restrict__ sinv, int T) {
    const int half = rotary_dim / 2;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)T * half) return;
    const int t = (int)(idx / half), j = (int)(idx % half);
    const float ang = (float)pos[t] / powf(theta, (float)(2 * j) / (float)rotary_dim);
    cosv[idx] = cosf(ang);
    sinv[idx] = sinf(ang);
}

extern "C" int li_rope_table(const int* pos, float theta, int rotary_dim, float* cosv, float* sinv,
                             int T, hipStream_t stream) {
    if (T <= 0 || rotary_dim <= 0 || (rotary_dim & 1)) return LI_ERR_SIZE;
    const long n = (long)T * (rotary_dim / 2);
    rope_table_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(pos, theta, rotary_dim, cosv, sinv, T);
    return li_launch_status();
}

// y[j] = a cos - b sin; y[j + half] = b cos + a sin with a = x[j], b = x[j + half]
// One rotation, with its roundings spelled out (one product rounded, the other fused into the sum),
// so that every kernel here gives the same bits whatever the compiler would contract.
__device__ __forceinline__ void rotate_values(float a, float b, float c, float s, float& ra, float& rb) {
    ra = __builtin_fmaf(a, c, -__fmul_rn(b, s));
    rb = __builtin_fmaf(b, c, __fmul_rn(a, s));
}

template <typename T>
__device__ __forceinline__ void rotate_pair(T* head, int j, int half, float c, float s, T* dst) {
    const float a = load_as_float(head + j), b = load_as_float(head + j + half);
    float ra, rb;
    rotate_values(a, b, c, s, ra, rb);
    store_from_float(dst + j, ra);
    store_from_float(dst + j + half, rb);
}

template <typename T>
__global__ void rope_apply_kernel(T* __restrict__ qkv, int row_stride, int head_dim, int rotary_dim,
                                  const float* __restrict__ cosv, const float* __restrict__ sinv) {
    const int t = blockIdx.x, h = blockIdx.y, half = rotary_dim / 2;
    T* head = qkv + (size_t)t * row_stride + (size_t)h * head_dim;
    for (int j = threadIdx.x; j < half; j += blockDim.x)
        rotate_pair(head, j, half, cosv[(size_t)t * half + j], sinv[(size_t)t * half + j], head);
}

extern "C" int li_rope_apply(void* qkv, int dtype, int row_stride, int n_heads, int head_dim,
                             int rotary_dim, const float* cosv, const float* sinv, int T,
                             hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || n_heads > 65535 || rotary_dim > head_dim || (rotary_dim & 1)) return LI_ERR_SIZE;
    dim3 grid(T, n_heads);
    if (dtype == LI_F32) rope_apply_kernel<float><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, head_dim, rotary_dim, cosv, sinv);
    else if (dtype == LI_BF16) rope_apply_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, head_dim, rotary_dim, cosv, sinv);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ----------------------------------------------------------------- kv store
// Cache layout per layer: [pages, kv_heads, page_size, head_dim]; the slot of
// a token is page * page_size + offset.
template <typename T>
__device__ __forceinline__ T* cache_row(T* base, int slot, int page_size, int nkv, int kvh, int dh) {
    const int page = slot / page_size, off = slot - page * page_size;
    return base + (((size_t)page * nkv + kvh) * page_size + off) * dh;
}

// grid (T, nh + 2 nkv) when ROTATE (query heads rotated in place, key heads
// rotated into the cache, value heads copied), grid (T, 2 nkv) otherwise
template <typename T, bool ROTATE>
__global__ void kv_store_kernel(T* __restrict__ qkv, int row_stride, int nh, int nkv, int dh,
                                int rotary_dim, const float* __restrict__ cosv,
                                const float* __restrict__ sinv, const int* __restrict__ slot_map,
                                T* __restrict__ kc, T* __restrict__ vc, int page_size, int num_pages) {
    const int t = blockIdx.x;
    int hh = blockIdx.y + (ROTATE ? 0 : nh);
    T* head = qkv + (size_t)t * row_stride + (size_t)hh * dh;
    const int half = rotary_dim / 2;
    if (hh < nh) {                                               // query head: rotate in place
        for (int j = threadIdx.x; j < half; j += blockDim.x)
            rotate_pair(head, j, half, cosv[(size_t)t * half + j], sinv[(size_t)t * half + j], head);
        return;
    }
    const int slot = slot_map[t];
    if (slot < 0 || slot >= num_pages * page_size) return;       // never write outside the pool
    if (hh < nh + nkv) {
        T* dst = cache_row(kc, slot, page_size, nkv, hh - nh, dh);
        if (ROTATE) {
            for (int j = threadIdx.x; j < half; j += blockDim.x)
                rotate_pair(head, j, half, cosv[(size_t)t * half + j], sinv[(size_t)t * half + j], dst);
            for (int j = rotary_dim + threadIdx.x; j < dh; j += blockDim.x) dst[j] = head[j];
        } else {
            for (int j = threadIdx.x; j < dh; j += blockDim.x) dst[j] = head[j];
        }
    } else {
        T* dst = cache_row(vc, slot, page_size, nkv, hh - nh - nkv, dh);
        for (int j = threadIdx.x; j < dh; j += blockDim.x) dst[j] = head[j];
    }
}

// The same with 16 bytes a lane, for whole-head rotation (rotary_dim == dh) or none, where a half
// head is a whole number of 16-byte pieces and rows start on 16 bytes: thread (t, head, c) takes
// the pieces c of the head's two halves, i.e. E pairs when it rotates.
template <typename T, bool ROTATE>
__global__ __launch_bounds__(256) void kv_store_vec_kernel(T* __restrict__ qkv, int row_stride, int nh, int nkv, int dh,
                                                            const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                            const int* __restrict__ slot_map, T* __restrict__ kc,
                                                            T* __restrict__ vc, int page_size, int num_pages, long total) {
    constexpr int E = 16 / (int)sizeof(T);
    struct __attribute__((aligned(16))) piece { T e[E]; };
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int half = dh / 2, cph = half / E;                     // pieces in half a head
    const int nheads = ROTATE ? nh + 2 * nkv : 2 * nkv;
    const int c = (int)(i % cph);
    const int hh = (int)((i / cph) % nheads) + (ROTATE ? 0 : nh);
    const int t = (int)(i / ((long)cph * nheads));
    T* head = qkv + (size_t)t * row_stride + (size_t)hh * dh;
    T* dst = head;                                               // query heads: rotated in place
    if (hh >= nh) {
        const int slot = slot_map[t];
        if (slot < 0 || slot >= num_pages * page_size) return;   // never write outside the pool
        dst = hh < nh + nkv ? cache_row(kc, slot, page_size, nkv, hh - nh, dh)
                            : cache_row(vc, slot, page_size, nkv, hh - nh - nkv, dh);
    }
    piece a = *reinterpret_cast<const piece*>(head + E * c), b = *reinterpret_cast<const piece*>(head + half + E * c);
    if (ROTATE && hh < nh + nkv) {
        const float* cs = cosv + (size_t)t * half + E * c;
        const float* sn = sinv + (size_t)t * half + E * c;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float ra, rb;
            rotate_values(load_as_float(&a.e[e]), load_as_float(&b.e[e]), cs[e], sn[e], ra, rb);
            store_from_float(&a.e[e], ra);
            store_from_float(&b.e[e], rb);
        }
    } else if (dst == head) {
        return;                                                  // (cannot happen: an unrotated head is a cache head)
    }
    *reinterpret_cast<piece*>(dst + E * c) = a;
    *reinterpret_cast<piece*>(dst + half + E * c) = b;
}

template <typename T, bool ROTATE>
static bool kv_store_vec(T* qkv, int row_stride, int nh, int nkv, int dh, int rotary_dim, const float* cosv,
                         const float* sinv, const int* slot_map, T* kc, T* vc, int page_size, int num_pages, int Tn,
                         hipStream_t stream) {
    constexpr int E = 16 / (int)sizeof(T);
    if ((ROTATE && rotary_dim != dh) || dh % (2 * E) || row_stride % E || ((uintptr_t)qkv | (uintptr_t)kc | (uintptr_t)vc) % 16 ||
        (ROTATE && (((uintptr_t)cosv | (uintptr_t)sinv) % 16)))
        return false;
    const long total = (long)Tn * (ROTATE ? nh + 2 * nkv : 2 * nkv) * (dh / 2 / E);
    const long blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffL) return false;
    kv_store_vec_kernel<T, ROTATE><<<(unsigned)blocks, 256, 0, stream>>>(qkv, row_stride, nh, nkv, dh, cosv, sinv, slot_map, kc, vc,
                                                                        page_size, num_pages, total);
    return true;
}

extern "C" int li_kv_store(void* qkv, int dtype, int row_stride, int nh, int nkv, int dh,
                           const int* slot_map, void* kc, void* vc, int page_size, int num_pages,
                           int T, hipStream_t stream) {
    if (T <= 0 || nkv <= 0 || 2 * nkv > 65535 || page_size <= 0) return LI_ERR_SIZE;
    dim3 grid(T, 2 * nkv);
    if (dtype == LI_F32 && kv_store_vec<float, false>((float*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (float*)kc, (float*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_BF16 && kv_store_vec<bf16_t, false>((bf16_t*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_F32) kv_store_kernel<float, false><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (float*)kc, (float*)vc, page_size, num_pages);
    else if (dtype == LI_BF16) kv_store_kernel<bf16_t, false><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

extern "C" int li_rope_kv_store(void* qkv, int dtype, int row_stride, int nh, int nkv, int dh,
                                int rotary_dim, const float* cosv, const float* sinv,
                                const int* slot_map, void* kc, void* vc, int page_size,
                                int num_pages, int T, hipStream_t stream) {
    if (T <= 0 || nh + 2 * nkv > 65535 || page_size <= 0 || rotary_dim > dh || (rotary_dim & 1)) return LI_ERR_SIZE;
    dim3 grid(T, nh + 2 * nkv);
    if (dtype == LI_F32 && kv_store_vec<float, true>((float*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (float*)kc, (float*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_BF16 && kv_store_vec<bf16_t, true>((bf16_t*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_F32) kv_store_kernel<float, true><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (float*)kc, (float*)vc, page_size, num_pages);
    else if (dtype == LI_BF16) kv_store_kernel<bf16_t, true><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ============================================================================================
// Parts that several designs share: a stream that takes a second gather and a vector, a norm whose
// result is ADDED to the stream (a norm behind a sublayer), squared ReLU, a tanh-GELU gate times a
// slice of a second embedding table, rotary tables from given frequencies, and the rotation of
// neighbouring pairs.
// ============================================================================================

// out[t, :] += (table ? table[id(t), :] : 0) + (vec ? vec[:] : 0), all in float32; ids as in embedding_kernel
template <typename T>
__global__ void embedding_add_kernel(const int* __restrict__ ids, const int* __restrict__ id_src,
                                     const int* __restrict__ feedback, const T* __restrict__ table,
                                     const float* __restrict__ vec, float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = -1;
    if (table) {                                   // (without a table no ids are given)
        id = ids[t];
        if (id_src) {
            const int src = id_src[t];
            if (src >= 0) id = feedback[src];
        }
    }
    float* o = out + (size_t)t * H;
    const T* row = (table && id >= 0 && id < V) ? table + (size_t)id * H : nullptr;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float v = o[j];
        if (row) v += load_as_float(row + j);
        if (vec) v += vec[j];
        o[j] = v;
    }
}

extern "C" int li_embedding_add(const int* ids, const int* id_src, const int* feedback, const void* table,
                                int table_dtype, const float* vec, float* out, int T, int H, int V, hipStream_t stream) {
    if (T <= 0 || H <= 0 || (id_src && !feedback) || (table && !ids)) return LI_ERR_SIZE;
    if (table_dtype == LI_F32)
        embedding_add_kernel<float><<<T, 256, 0, stream>>>(ids, id_src, feedback, (const float*)table, vec, out, H, V);
    else if (table_dtype == LI_BF16)
        embedding_add_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, id_src, feedback, (const bf16_t*)table, vec, out, H, V);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// x[t, :] += b / sqrt(mean(b^2) + eps) * w for the branch b = y (or, with y2, b = a1 y + a2 y2), and, for whoever
// reads the stream next, xn[t, :] = the RMS norm of the NEW x with weights w2 and eps2 (next 1) or the new x itself in
// xn's type (next 2): one block a row.
template <typename TO, int NT>
__global__ __launch_bounds__(NT) void rmsnorm_add_kernel(const float* __restrict__ y, const float* __restrict__ y2, float a1, float a2,
                                                          const float* __restrict__ w, float eps,
                                                          float* __restrict__ x, const float* __restrict__ w2, float eps2,
                                                          TO* __restrict__ xn, int next, int H) {
    __shared__ float red[NT / LI_WAVE];
    const float* yr = y + (size_t)blockIdx.x * H;
    const float* yr2 = y2 ? y2 + (size_t)blockIdx.x * H : nullptr;
    float* xr = x + (size_t)blockIdx.x * H;
    float ss = 0.f;
    for (int j = threadIdx.x; j < H; j += NT) { const float v = yr2 ? a1 * yr[j] + a2 * yr2[j] : yr[j]; ss += v * v; }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    float s2 = 0.f;
    for (int j = threadIdx.x; j < H; j += NT) {
        const float b = yr2 ? a1 * yr[j] + a2 * yr2[j] : yr[j];
        const float v = xr[j] + b * inv * w[j];
        xr[j] = v;
        s2 += v * v;
    }
    if (next == 0) return;
    TO* o = xn + (size_t)blockIdx.x * H;
    if (next == 2) {
        for (int j = threadIdx.x; j < H; j += NT) store_from_float(o + j, xr[j]);               // (a thread reads back what it wrote)
        return;
    }
    s2 = block_sum<NT>(s2, red);
    const float inv2 = 1.0f / sqrtf(s2 / (float)H + eps2);
    for (int j = threadIdx.x; j < H; j += NT) store_from_float(o + j, xr[j] * inv2 * w2[j]);
}

extern "C" int li_rmsnorm_add(const float* y, const float* y2, float a1, float a2, const float* w, float eps, float* x,
                              const float* w2, float eps2, void* xn, int xn_dtype, int next, int T, int H, hipStream_t stream) {
    if (T <= 0 || H <= 0 || next < 0 || next > 2) return LI_ERR_SIZE;
    if ((next && !xn) || (next == 1 && !w2)) return LI_ERR_SIZE;
    const bool wide = T < 256 && H > 1024;
#define LI_RA(TO)                                                                                             \
    {                                                                                                         \
        if (wide) rmsnorm_add_kernel<TO, 1024><<<T, 1024, 0, stream>>>(y, y2, a1, a2, w, eps, x, w2, eps2, (TO*)xn, next, H);   \
        else rmsnorm_add_kernel<TO, 256><<<T, 256, 0, stream>>>(y, y2, a1, a2, w, eps, x, w2, eps2, (TO*)xn, next, H);          \
    }
    if (!next || xn_dtype == LI_F32) LI_RA(float)
    else if (xn_dtype == LI_BF16) LI_RA(bf16_t)
    else return LI_ERR_DTYPE;
#undef LI_RA
    return li_launch_status();
}

// out = max(x, 0)^2
template <typename TI, typename TO>
__global__ void relu_squared_kernel(const TI* __restrict__ x, TO* __restrict__ out, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = fmaxf(load_as_float(x + i), 0.f);
        store_from_float(out + i, v * v);
    }
}

extern "C" int li_relu_squared(const void* x, int x_dtype, void* out, int out_dtype, long n, hipStream_t stream) {
    if (n <= 0) return LI_ERR_SIZE;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (x_dtype == LI_F32 && out_dtype == LI_F32) relu_squared_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)x, (float*)out, n);
    else if (x_dtype == LI_F32 && out_dtype == LI_BF16) relu_squared_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((const float*)x, (bf16_t*)out, n);
    else if (x_dtype == LI_BF16 && out_dtype == LI_BF16) relu_squared_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, n);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

__device__ __forceinline__ float gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// out[t, j] = gelu_tanh(a[t, j]) * table[id(t), off + j], j < n; table rows have `row` elements
template <typename TT, typename TO>
__global__ void gelu_gate_rows_kernel(const float* __restrict__ a, const int* __restrict__ ids, const int* __restrict__ id_src,
                                      const int* __restrict__ feedback, const TT* __restrict__ table, int row, int off, int V,
                                      TO* __restrict__ out, int n) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id_src) {
        const int src = id_src[t];
        if (src >= 0) id = feedback[src];
    }
    const bool ok = id >= 0 && id < V;
    const TT* e = table + (size_t)(ok ? id : 0) * row + off;
    for (int j = threadIdx.x; j < n; j += blockDim.x)
        store_from_float(out + (size_t)t * n + j, ok ? gelu_tanh(a[(size_t)t * n + j]) * load_as_float(e + j) : 0.f);
}

extern "C" int li_gelu_gate_rows(const float* a, const int* ids, const int* id_src, const int* feedback, const void* table,
                                 int table_dtype, int row, int off, int V, void* out, int out_dtype, int T, int n,
                                 hipStream_t stream) {
    if (T <= 0 || n <= 0 || off < 0 || off + n > row || (id_src && !feedback)) return LI_ERR_SIZE;
    const int nt = n >= 256 ? 256 : 64;
#define LI_GG(TT, TO) gelu_gate_rows_kernel<TT, TO><<<T, nt, 0, stream>>>(a, ids, id_src, feedback, (const TT*)table, row, off, V, (TO*)out, n)
    if (table_dtype == LI_F32 && out_dtype == LI_F32) LI_GG(float, float);
    else if (table_dtype == LI_BF16 && out_dtype == LI_BF16) LI_GG(bf16_t, bf16_t);
    else if (table_dtype == LI_BF16 && out_dtype == LI_F32) LI_GG(bf16_t, float);
    else if (table_dtype == LI_F32 && out_dtype == LI_BF16) LI_GG(float, bf16_t);
    else return LI_ERR_DTYPE;
#undef LI_GG
    return li_launch_status();
}

// cos/sin [T, n] of angle = float(pos[t]) * freq[i], each times `amp`: the frequencies are given
// (whatever scaling they went through on the host), the product and the functions are float32
__global__ void rope_freq_table_kernel(const int* __restrict__ pos, const float* __restrict__ freq, int n, float amp,
                                       float* __restrict__ cosv, float* __restrict__ sinv, int T) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)T * n) return;
    const int t = (int)(idx / n), i = (int)(idx % n);
    const float ang = (float)pos[t] * freq[i];
    cosv[idx] = cosf(ang) * amp;
    sinv[idx] = sinf(ang) * amp;
}

extern "C" int li_rope_freq_table(const int* pos, const float* freq, int n, float amp, float* cosv, float* sinv, int T,
                                  hipStream_t stream) {
    if (T <= 0 || n <= 0) return LI_ERR_SIZE;
    const long total = (long)T * n;
    rope_freq_table_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(pos, freq, n, amp, cosv, sinv, T);
    return li_launch_status();
}

// neighbouring pairs: (u, v) = (x[2i], x[2i+1]) -> (u cos - v sin, v cos + u sin)
__device__ __forceinline__ void rotate_pair(float u, float v, float c, float s, float& ru, float& rv) {
    ru = fmaf(u, c, -__fmul_rn(v, s));
    rv = fmaf(v, c, __fmul_rn(u, s));
}

// in place, heads 0..n_heads-1 of every row (head h at columns h * head_dim ..), the first rotary_dim of each
template <typename T>
__global__ void rope_pairs_apply_kernel(T* __restrict__ x, int row_stride, int n_heads, int head_dim, int rotary_dim,
                                        const float* __restrict__ cosv, const float* __restrict__ sinv) {
    const int t = blockIdx.x, half = rotary_dim / 2;
    T* row = x + (size_t)t * row_stride;
    for (int u = threadIdx.x; u < n_heads * half; u += blockDim.x) {
        const int h = u / half, i = u % half;
        T* p = row + (size_t)h * head_dim + 2 * i;
        float a, b;
        rotate_pair(load_as_float(p), load_as_float(p + 1), cosv[(size_t)t * half + i], sinv[(size_t)t * half + i], a, b);
        store_from_float(p, a);
        store_from_float(p + 1, b);
    }
}

extern "C" int li_rope_pairs_apply(void* x, int dtype, int row_stride, int n_heads, int head_dim, int rotary_dim,
                                   const float* cosv, const float* sinv, int T, hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || rotary_dim <= 0 || (rotary_dim & 1) || rotary_dim > head_dim) return LI_ERR_SIZE;
    if (dtype == LI_F32) rope_pairs_apply_kernel<float><<<T, 256, 0, stream>>>((float*)x, row_stride, n_heads, head_dim, rotary_dim, cosv, sinv);
    else if (dtype == LI_BF16) rope_pairs_apply_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)x, row_stride, n_heads, head_dim, rotary_dim, cosv, sinv);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// The step between the packed q/k/v projection (float32 rows [q | k | v]) and the attention, for a mixer that
// norms the WHOLE query projection and the WHOLE key projection (all heads at once, before they are split) and
// rotates pairs of columns (neighbours, or with half_split column i and column i + rotary_dim / 2): q is normed and rotated in place (it stays float32), k is normed, rotated and
// written to its page slot, v is copied to its page slot.  wq / wk null: no norm.  One block a token.
template <typename T, int NT>
__global__ __launch_bounds__(NT) void qk_norm_pairs_store_kernel(
    float* __restrict__ qkv, int row_stride, int nh, int nkv, int dk, int dv, int rotary_dim,
    const float* __restrict__ wq, const float* __restrict__ wk, float eps,
    const float* __restrict__ cosv, const float* __restrict__ sinv, const int* __restrict__ slot_map,
    T* __restrict__ kc, T* __restrict__ vc, int page_size, int store, int half_split) {
    __shared__ float red[NT / LI_WAVE];
    const int t = blockIdx.x, half = rotary_dim / 2;
    float* q = qkv + (size_t)t * row_stride;
    float* k = q + (size_t)nh * dk;
    const float* v = k + (size_t)nkv * dk;
    const int nq = nh * dk, nk = nkv * dk;
    float inv_q = 1.f, inv_k = 1.f;
    if (wq) {
        float s = 0.f;
        for (int j = threadIdx.x; j < nq; j += NT) s += q[j] * q[j];
        s = block_sum<NT>(s, red);
        inv_q = 1.0f / sqrtf(s / (float)nq + eps);
    }
    if (wk && store) {
        float s = 0.f;
        for (int j = threadIdx.x; j < nk; j += NT) s += k[j] * k[j];
        s = block_sum<NT>(s, red);
        inv_k = 1.0f / sqrtf(s / (float)nk + eps);
    }
    const float* c = cosv + (size_t)t * half;
    const float* sn = sinv + (size_t)t * half;
    const int units = half + (dk - rotary_dim);            // per head: the pairs, then the columns that are not rotated
    for (int u = threadIdx.x; u < nh * units; u += NT) {
        const int h = u / units, i = u % units;
        if (i < half) {
            const int j = h * dk + (half_split ? i : 2 * i), j2 = half_split ? j + half : j + 1;    // the pair's two columns
            const float a = wq ? q[j] * inv_q * wq[j] : q[j], b = wq ? q[j2] * inv_q * wq[j2] : q[j2];
            float ra, rb;
            rotate_pair(a, b, c[i], sn[i], ra, rb);
            q[j] = ra; q[j2] = rb;
        } else if (wq) {
            const int j = h * dk + rotary_dim + (i - half);
            q[j] = q[j] * inv_q * wq[j];
        }
    }
    if (!store) return;
    const int slot = slot_map[t], page = slot / page_size, off = slot % page_size;
    for (int u = threadIdx.x; u < nkv * units; u += NT) {
        const int h = u / units, i = u % units;
        T* dst = kc + ((size_t)(page * nkv + h) * page_size + off) * dk;
        if (i < half) {
            const int d1 = half_split ? i : 2 * i, d2 = half_split ? i + half : 2 * i + 1;
            const int j = h * dk + d1, j2 = h * dk + d2;
            const float a = wk ? k[j] * inv_k * wk[j] : k[j], b = wk ? k[j2] * inv_k * wk[j2] : k[j2];
            float ra, rb;
            rotate_pair(a, b, c[i], sn[i], ra, rb);
            store_from_float(dst + d1, ra);
            store_from_float(dst + d2, rb);
        } else {
            const int d = rotary_dim + (i - half), j = h * dk + d;
            store_from_float(dst + d, wk ? k[j] * inv_k * wk[j] : k[j]);
        }
    }
    for (int u = threadIdx.x; u < nkv * dv; u += NT) {
        const int h = u / dv, d = u % dv;
        store_from_float(vc + ((size_t)(page * nkv + h) * page_size + off) * dv + d, v[u]);
    }
}

extern "C" int li_qk_norm_pairs_store(float* qkv, int row_stride, int nh, int nkv, int dk, int dv, int rotary_dim,
                                      const float* wq, const float* wk, float eps, const float* cosv, const float* sinv,
                                      const int* slot_map, void* kc, void* vc, int cache_dtype, int page_size, int store,
                                      int half_split, int T, hipStream_t stream) {
    if (T <= 0 || nh <= 0 || nkv <= 0 || dk <= 0 || dv <= 0 || rotary_dim < 0 || (rotary_dim & 1) || rotary_dim > dk ||
        row_stride < nh * dk + nkv * (dk + dv) || page_size <= 0)
        return LI_ERR_SIZE;
    // few rows (a decoding step): 1024 threads a row, so that the one row is gone through with the least latency
    const bool wide = T < 256 && nh * dk > 1024;
#define LI_QK(TC)                                                                                                            \
    {                                                                                                                        \
        if (wide) qk_norm_pairs_store_kernel<TC, 1024><<<T, 1024, 0, stream>>>(qkv, row_stride, nh, nkv, dk, dv, rotary_dim, wq, wk, eps, \
                                                                              cosv, sinv, slot_map, (TC*)kc, (TC*)vc, page_size, store, half_split); \
        else qk_norm_pairs_store_kernel<TC, 256><<<T, 256, 0, stream>>>(qkv, row_stride, nh, nkv, dk, dv, rotary_dim, wq, wk, eps,  \
                                                                        cosv, sinv, slot_map, (TC*)kc, (TC*)vc, page_size, store, half_split);  \
    }
    if (cache_dtype == LI_F32) LI_QK(float)
    else if (cache_dtype == LI_BF16) LI_QK(bf16_t)
    else return LI_ERR_DTYPE;
#undef LI_QK
    return li_launch_status();
}

// The same step for attention over a compressed cache.  `q` (float32 rows, may be absent: nh = 0) holds nh heads of
// (dn + dr) columns, the last dr of each rotated; `down` (float32 rows, which may lie inside the same buffer) holds
// `rank` latent columns and dr columns of one rotated key part that all heads share.  The latent is RMS-normed
// (weights wc) and written to columns 0..rank-1 of the token's page row, the rotated shared part behind it; the
// rotated part of every query head goes to columns rank.. of that head's row in `qfull` (float32 rows of
// nh x (rank + dr): the first `rank` columns are filled by the product with the keys' expansion matrix afterwards).
// `split`: 0 pairs neighbouring columns (2i, 2i + 1), 1 pairs column i with column i + dr/2.
// Where the queries go through a latent of their own, `ql` holds its q_rank columns before the norm and `cq` takes
// the RMS norm with weights wq (in the dtype of the product that follows).
template <typename T, typename TQ, int NT>
__global__ __launch_bounds__(NT) void latent_norm_pairs_store_kernel(
    const float* __restrict__ q, long q_stride, int nh, int dn, int dr, const float* __restrict__ down, long down_stride,
    int rank, const float* __restrict__ wc, float eps, const float* __restrict__ cosv, const float* __restrict__ sinv,
    const int* __restrict__ slot_map, T* __restrict__ cache, float* __restrict__ qfull, int store, int split,
    const float* __restrict__ ql, long ql_stride, int q_rank, const float* __restrict__ wq, TQ* __restrict__ cq) {
    __shared__ float red[NT / LI_WAVE];
    const int t = blockIdx.x, half = dr / 2;
    const int second = split ? half : 1, step = split ? 1 : 2;       // a pair is (step * i, step * i + second)
    const float* c = cosv + (size_t)t * half;
    const float* sn = sinv + (size_t)t * half;
    if (nh > 0) {
        const float* qr = q + (size_t)t * q_stride;
        float* qf = qfull + (size_t)t * nh * (rank + dr);
        for (int u = threadIdx.x; u < nh * half; u += NT) {
            const int h = u / half, i = u % half;
            const float* src = qr + (size_t)h * (dn + dr) + dn + step * i;
            float ra, rb;
            rotate_pair(src[0], src[second], c[i], sn[i], ra, rb);
            float* dst = qf + (size_t)h * (rank + dr) + rank + step * i;
            dst[0] = ra; dst[second] = rb;
        }
    }
    if (q_rank > 0) {
        const float* lr = ql + (size_t)t * ql_stride;
        float s = 0.f;
        for (int j = threadIdx.x; j < q_rank; j += NT) s += lr[j] * lr[j];
        s = block_sum<NT>(s, red);
        const float inv = 1.0f / sqrtf(s / (float)q_rank + eps);
        TQ* o = cq + (size_t)t * q_rank;
        for (int j = threadIdx.x; j < q_rank; j += NT) store_from_float(o + j, wq[j] * lr[j] * inv);
    }
    if (!store) return;
    const float* dw = down + (size_t)t * down_stride;
    float s = 0.f;
    for (int j = threadIdx.x; j < rank; j += NT) s += dw[j] * dw[j];
    s = block_sum<NT>(s, red);
    const float inv = 1.0f / sqrtf(s / (float)rank + eps);
    T* row = cache + (size_t)slot_map[t] * (rank + dr);
    for (int j = threadIdx.x; j < rank; j += NT) store_from_float(row + j, dw[j] * inv * wc[j]);
    for (int i = threadIdx.x; i < half; i += NT) {
        float ra, rb;
        rotate_pair(dw[rank + step * i], dw[rank + step * i + second], c[i], sn[i], ra, rb);
        store_from_float(row + rank + step * i, ra);
        store_from_float(row + rank + step * i + second, rb);
    }
}

extern "C" int li_latent_norm_pairs_store(const float* q, long q_stride, int nh, int dn, int dr, const float* down,
                                          long down_stride, int rank, const float* wc, float eps, const float* cosv,
                                          const float* sinv, const int* slot_map, void* cache, int cache_dtype, float* qfull,
                                          int store, int split, const float* ql, long ql_stride, int q_rank, const float* wq,
                                          void* cq, int cq_dtype, int T, hipStream_t stream) {
    if (T <= 0 || nh < 0 || dn < 0 || dr <= 0 || (dr & 1) || rank <= 0 || q_rank < 0) return LI_ERR_SIZE;
    if ((nh > 0 && (!q || !qfull || q_stride < (long)nh * (dn + dr))) || (store && (!down || !cache || !slot_map || down_stride < rank + dr)) ||
        (q_rank > 0 && (!ql || !wq || !cq || ql_stride < q_rank)))
        return LI_ERR_SIZE;
#define LI_LN(T_, TQ_)                                                                                                          \
    latent_norm_pairs_store_kernel<T_, TQ_, 256><<<T, 256, 0, stream>>>(q, q_stride, nh, dn, dr, down, down_stride, rank, wc, eps, \
                                                                        cosv, sinv, slot_map, (T_*)cache, qfull, store, split, ql, \
                                                                        ql_stride, q_rank, wq, (TQ_*)cq)
    if (cache_dtype == LI_F32 && cq_dtype == LI_F32) LI_LN(float, float);
    else if (cache_dtype == LI_BF16 && cq_dtype == LI_BF16) LI_LN(bf16_t, bf16_t);
    else if (cache_dtype == LI_F32 && cq_dtype == LI_BF16) LI_LN(float, bf16_t);
    else if (cache_dtype == LI_BF16 && cq_dtype == LI_F32) LI_LN(bf16_t, float);
    else return LI_ERR_DTYPE;
#undef LI_LN
    return li_launch_status();
}

// ------------------------------------------------------------------------------ sinusoidal position vector
// x[t, 2i] += sin(p f_i), x[t, 2i + 1] += cos(p f_i) with p = positions[t] and f the table of frequencies
// (worked out by the caller, one per pair of columns); the angle is float(p) * f_i in float32.
__global__ void sinusoid_add_kernel(float* __restrict__ x, const int* __restrict__ positions, const float* __restrict__ freq, int H) {
    const int t = blockIdx.x;
    const float p = (float)positions[t];
    float* row = x + (size_t)t * H;
    for (int i = threadIdx.x; 2 * i < H; i += blockDim.x) {
        const float a = p * freq[i];
        row[2 * i] += sinf(a);
        if (2 * i + 1 < H) row[2 * i + 1] += cosf(a);
    }
}

extern "C" int li_sinusoid_add(float* x, const int* positions, const float* freq, int T, int H, hipStream_t stream) {
    if (T <= 0 || H <= 0) return LI_ERR_SIZE;
    sinusoid_add_kernel<<<T, 256, 0, stream>>>(x, positions, freq, H);
    return li_launch_status();
}

// ------------------------------------------------------------------------------ scaled and capped logits
// v <- v * scale, then, where cap > 0, cap * tanh(v / cap)
__global__ void scale_softcap_kernel(float* __restrict__ x, long n, float scale, float cap) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = x[i] * scale;
        x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
    }
}

extern "C" int li_scale_softcap(float* x, long n, float scale, float cap, hipStream_t stream) {
    if (n <= 0 || cap < 0.f) return LI_ERR_SIZE;
    scale_softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, n, scale, cap);
    return li_launch_status();
}

// ------------------------------------------------------------------------------ columns of rows into pages
// Up to three runs of columns of a float32 row (run r: `heads[r]` heads of `dim[r]` columns from column col[r] on) go to
// the token's slot in three paged tensors [pages, heads, page_size, dim].
struct PagedRuns { int col[3]; int heads[3]; int dim[3]; void* dst[3]; };

template <typename T>
__global__ void paged_store_kernel(const float* __restrict__ src, long stride, PagedRuns runs, const int* __restrict__ slot_map,
                                   int page_size) {
    const int t = blockIdx.x;
    const int slot = slot_map[t], page = slot / page_size, off = slot % page_size;
    const float* row = src + (size_t)t * stride;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const int nh = runs.heads[r], d = runs.dim[r];
        T* dst = (T*)runs.dst[r];
        for (int u = threadIdx.x; u < nh * d; u += blockDim.x) {
            const int h = u / d, j = u % d;
            store_from_float(dst + ((size_t)(page * nh + h) * page_size + off) * d + j, row[runs.col[r] + u]);
        }
    }
}

extern "C" int li_paged_store(const float* src, long stride, int col0, int heads0, int dim0, void* dst0, int col1, int heads1,
                              int dim1, void* dst1, int col2, int heads2, int dim2, void* dst2, int cache_dtype,
                              const int* slot_map, int page_size, int T, hipStream_t stream) {
    if (T <= 0 || page_size <= 0 || heads0 < 0 || heads1 < 0 || heads2 < 0 || dim0 < 0 || dim1 < 0 || dim2 < 0) return LI_ERR_SIZE;
    PagedRuns runs{{col0, col1, col2}, {heads0, heads1, heads2}, {dim0, dim1, dim2}, {dst0, dst1, dst2}};
    for (int r = 0; r < 3; ++r)
        if (runs.heads[r] && (runs.col[r] < 0 || runs.col[r] + (long)runs.heads[r] * runs.dim[r] > stride || !runs.dst[r])) return LI_ERR_SIZE;
    if (cache_dtype == LI_F32) paged_store_kernel<float><<<T, 256, 0, stream>>>(src, stride, runs, slot_map, page_size);
    else if (cache_dtype == LI_BF16) paged_store_kernel<bf16_t><<<T, 256, 0, stream>>>(src, stride, runs, slot_map, page_size);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ------------------------------------------------------------------------------ difference of two attention maps
// o = a1 - lambda * a2 per (token, head), then o / sqrt(mean(o^2) + eps) over the head's columns, times `mult`.
// A wave a (token, head).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void diff_combine_kernel(const TI* __restrict__ a1, const TI* __restrict__ a2, float lambda,
                                                           float eps, float mult, TO* __restrict__ out, long pairs, int dv) {
    const long pr = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pr >= pairs) return;
    const int lane = threadIdx.x & 63;
    const TI* r1 = a1 + (size_t)pr * dv;
    const TI* r2 = a2 + (size_t)pr * dv;
    float ss = 0.f;
    for (int j = lane; j < dv; j += 64) {
        const float o = fmaf(-lambda, load_as_float(r2 + j), load_as_float(r1 + j));
        ss = fmaf(o, o, ss);
    }
    ss = wave_sum(ss);
    const float f = mult / sqrtf(ss / (float)dv + eps);
    for (int j = lane; j < dv; j += 64) {
        const float o = fmaf(-lambda, load_as_float(r2 + j), load_as_float(r1 + j));
        store_from_float(out + (size_t)pr * dv + j, o * f);
    }
}

extern "C" int li_diff_combine(const void* a1, const void* a2, int in_dtype, float lambda, float eps, float mult, void* out,
                               int out_dtype, long pairs, int dv, hipStream_t stream) {
    if (pairs <= 0 || dv <= 0) return LI_ERR_SIZE;
    const unsigned grid = (unsigned)((pairs + 3) / 4);
#define DC(TI, TO) diff_combine_kernel<TI, TO><<<grid, 256, 0, stream>>>((const TI*)a1, (const TI*)a2, lambda, eps, mult, (TO*)out, pairs, dv)
    if (in_dtype == LI_F32 && out_dtype == LI_F32) DC(float, float);
    else if (in_dtype == LI_F32 && out_dtype == LI_BF16) DC(float, bf16_t);
    else if (in_dtype == LI_BF16 && out_dtype == LI_BF16) DC(bf16_t, bf16_t);
    else if (in_dtype == LI_BF16 && out_dtype == LI_F32) DC(bf16_t, float);
    else return LI_ERR_DTYPE;
#undef DC
    return li_launch_status();
}

// ============================================================================================
// A hashed pair-of-tokens embedding, layer norm with bias, the tanh form of GELU, two rows side by side.
// ============================================================================================

// out[t, :] = table[id(t), :] + pair[row(t), :] in float32.  row(t) is (prev * mul_prev + id * mul_cur) mod buckets
// with prev the id of the token before t in its request, and row number `buckets` (the table's last) for a
// request's first token (position 0) or where an id is no token of the vocabulary.  The token before a step's first
// one of a request comes from `last[slot]`, which the same block then sets to the id of the request's last token of
// this step: one block a segment touches a slot, and it reads before it writes.
template <typename T>
__global__ void pair_embedding_kernel(const int* __restrict__ ids, const int* __restrict__ id_src,
                                      const int* __restrict__ feedback, const int* __restrict__ positions,
                                      const int* __restrict__ seg_of_token, const int* __restrict__ q_start,
                                      const int* __restrict__ q_len, const int* __restrict__ slots, int* __restrict__ last,
                                      const T* __restrict__ table, const T* __restrict__ pair, float* __restrict__ out,
                                      int H, int V, int buckets, long mul_prev, long mul_cur) {
    const int t = blockIdx.x;
    __shared__ int sid, sprev;
    if (threadIdx.x == 0) {
        auto id_of = [&](int u) {
            int id = ids[u];
            if (id_src) {
                const int src = id_src[u];
                if (src >= 0) id = feedback[src];
            }
            return id;
        };
        const int seg = seg_of_token[t], first = q_start[seg];
        const int id = id_of(t);
        int prev = -1;
        if (positions[t] > 0) prev = (t > first) ? id_of(t - 1) : last[slots[seg]];
        if (t == first) last[slots[seg]] = id_of(first + q_len[seg] - 1);
        sid = id; sprev = prev;
    }
    __syncthreads();
    const int id = sid, prev = sprev;
    const bool ok = id >= 0 && id < V;
    int row = buckets;
    if (ok && prev >= 0 && prev < V) row = (int)(((long)prev * mul_prev + (long)id * mul_cur) % (long)buckets);
    const T* e = table + (size_t)(ok ? id : 0) * H;
    const T* p = pair + (size_t)row * H;
    float* o = out + (size_t)t * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x)
        o[j] = (ok ? load_as_float(e + j) : 0.f) + load_as_float(p + j);
}

extern "C" int li_pair_embedding(const int* ids, const int* id_src, const int* feedback, const int* positions,
                                 const int* seg_of_token, const int* q_start, const int* q_len, const int* slots, int* last,
                                 const void* table, const void* pair, int table_dtype, float* out, int T, int H, int V,
                                 int buckets, long mul_prev, long mul_cur, hipStream_t stream) {
    if (T <= 0 || H <= 0 || V <= 0 || buckets <= 0 || mul_prev < 0 || mul_cur < 0 || (id_src && !feedback)) return LI_ERR_SIZE;
    if (table_dtype == LI_F32)
        pair_embedding_kernel<float><<<T, 256, 0, stream>>>(ids, id_src, feedback, positions, seg_of_token, q_start, q_len, slots,
                                                            last, (const float*)table, (const float*)pair, out, H, V, buckets,
                                                            mul_prev, mul_cur);
    else if (table_dtype == LI_BF16)
        pair_embedding_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, id_src, feedback, positions, seg_of_token, q_start, q_len, slots,
                                                             last, (const bf16_t*)table, (const bf16_t*)pair, out, H, V, buckets,
                                                             mul_prev, mul_cur);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b, one block a row; the row stays in registers (up to
// PER elements a thread, longer rows are read again), mean and variance are two passes over it, all in float32.
template <typename TO, int NT, int PER>
__global__ __launch_bounds__(NT) void layernorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, float eps, TO* __restrict__ out, int H) {
    __shared__ float red[NT / LI_WAVE];
    const float* row = x + (size_t)blockIdx.x * H;
    TO* o = out + (size_t)blockIdx.x * H;
    float v[PER];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        v[i] = (j < H) ? row[j] : 0.f;
        s += v[i];
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT) s += row[j];
    const float mean = block_sum<NT>(s, red) / (float)H;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        const float d = (j < H) ? v[i] - mean : 0.f;
        ss += d * d;
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT) { const float d = row[j] - mean; ss += d * d; }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        if (j < H) store_from_float(o + j, fmaf((v[i] - mean) * inv, w[j], b ? b[j] : 0.f));
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT)
        store_from_float(o + j, fmaf((row[j] - mean) * inv, w[j], b ? b[j] : 0.f));
}

extern "C" int li_layernorm(const float* x, const float* w, const float* b, float eps, void* out, int out_dtype, int T, int H,
                            hipStream_t stream) {
    if (T <= 0 || H <= 0) return LI_ERR_SIZE;
#define LI_LNORM(TO)                                                                                        \
    {                                                                                                       \
        if (T >= 256 || H <= 1024) layernorm_kernel<TO, 256, 16><<<T, 256, 0, stream>>>(x, w, b, eps, (TO*)out, H); \
        else layernorm_kernel<TO, 1024, 8><<<T, 1024, 0, stream>>>(x, w, b, eps, (TO*)out, H);              \
    }
    if (out_dtype == LI_F32) LI_LNORM(float)
    else if (out_dtype == LI_BF16) LI_LNORM(bf16_t)
    else return LI_ERR_DTYPE;
#undef LI_LNORM
    return li_launch_status();
}

// out = gelu_tanh(x), element by element
template <typename TI, typename TO>
__global__ void gelu_tanh_kernel(const TI* __restrict__ x, TO* __restrict__ out, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) store_from_float(out + i, gelu_tanh(load_as_float(x + i)));
}

extern "C" int li_gelu_tanh(const void* x, int x_dtype, void* out, int out_dtype, long n, hipStream_t stream) {
    if (n <= 0) return LI_ERR_SIZE;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (x_dtype == LI_F32 && out_dtype == LI_F32) gelu_tanh_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)x, (float*)out, n);
    else if (x_dtype == LI_F32 && out_dtype == LI_BF16) gelu_tanh_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((const float*)x, (bf16_t*)out, n);
    else if (x_dtype == LI_BF16 && out_dtype == LI_BF16) gelu_tanh_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, n);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// out[t, :] = [a[t, :] | b[t, :]] for float32 rows a and b of H columns, in the dtype of out
template <typename TO>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, TO* __restrict__ out, int H) {
    const int t = blockIdx.x;
    TO* o = out + (size_t)t * 2 * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        store_from_float(o + j, a[(size_t)t * H + j]);
        store_from_float(o + H + j, b[(size_t)t * H + j]);
    }
}

extern "C" int li_concat_rows(const float* a, const float* b, void* out, int out_dtype, int T, int H, hipStream_t stream) {
    if (T <= 0 || H <= 0) return LI_ERR_SIZE;
    if (out_dtype == LI_F32) concat_rows_kernel<float><<<T, 256, 0, stream>>>(a, b, (float*)out, H);
    else if (out_dtype == LI_BF16) concat_rows_kernel<bf16_t><<<T, 256, 0, stream>>>(a, b, (bf16_t*)out, H);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}
