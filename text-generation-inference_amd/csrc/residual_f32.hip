// Kernels around an fp32 residual stream: scaled embedding lookup, the "sandwich" RMS norm (norm after a sublayer, add,
// norm before the next one, in one launch) and gated-unit activations with optional clamping.
//
// Models that keep their residual stream in the model dtype use norm.hip; a design that asks for a 32-bit residual sum and
// norms on both sides of every sublayer uses these.  Activations handed to / taken from the matrix products are T = bf16,
// f16 or float; statistics, gains and the residual itself are always float.
#include "common.h"

namespace {

template <typename T> struct Elem;
template <> struct Elem<f16> { static __device__ __forceinline__ float ld(const f16* p) { return (float)*p; } };
template <> struct Elem<bf16> { static __device__ __forceinline__ float ld(const bf16* p) { return (float)*p; } };
template <> struct Elem<float> { static __device__ __forceinline__ float ld(const float* p) { return *p; } };
template <typename T> __device__ __forceinline__ T cvt_out(float v) { return (T)v; }

__device__ __forceinline__ float block_sum(float v, float* red) {
    // every thread of the block calls this; red holds one float per wave (<= 16)
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();  // red may still be read from a previous call
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}

template <typename T>
__global__ void embedding_scaled_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out,
                                        int64_t E, int64_t vocab, float scale) {
    const int64_t t = blockIdx.x;
    const int64_t id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    for (int64_t c = threadIdx.x; c < E; c += blockDim.x)
        out[t * E + c] = ok ? Elem<T>::ld(table + id * E + c) * scale : 0.f;
}

// One workgroup per row.
//   delta != null:  x_out = x + delta / sqrt(mean(delta^2) + eps) * (post_w + post_add)
//   pre_w != null:  y = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)
// x_out may alias x.  TD: dtype of delta, TY: dtype of y.
template <typename TD, typename TY>
__global__ __launch_bounds__(256) void sandwich_norm_kernel(const float* x, const TD* __restrict__ delta,
                                                            int64_t ld_delta, const float* __restrict__ post_w, float post_add,
                                                            float* x_out, const float* __restrict__ pre_w,
                                                            float pre_add, TY* __restrict__ y, int64_t E, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const float* xr = x + row * E;
    float* xo = x_out + row * E;
    float rinv_d = 0.f;
    if (delta) {
        const TD* dr = delta + row * ld_delta;
        float ss = 0.f;
        for (int64_t c = threadIdx.x; c < E; c += blockDim.x) {
            float d = Elem<TD>::ld(dr + c);
            ss += d * d;
        }
        ss = block_sum(ss, red);
        rinv_d = 1.0f / sqrtf(ss / (float)E + eps);
    }
    float ss2 = 0.f;
    for (int64_t c = threadIdx.x; c < E; c += blockDim.x) {
        float v = xr[c];
        if (delta) {
            v += Elem<TD>::ld(delta + row * ld_delta + c) * rinv_d * (post_w[c] + post_add);
            xo[c] = v;
        } else if (xo != xr) {
            xo[c] = v;
        }
        ss2 += v * v;
    }
    if (!pre_w) return;
    ss2 = block_sum(ss2, red);
    const float rinv = 1.0f / sqrtf(ss2 / (float)E + eps);
    for (int64_t c = threadIdx.x; c < E; c += blockDim.x) {
        // the same thread wrote xo[c] above
        float v = (delta || xo != xr) ? xo[c] : xr[c];
        y[row * E + c] = cvt_out<TY>(v * rinv * (pre_w[c] + pre_add));
    }
}


// The same, for E <= 256 * NPT: a row lives in registers, every global load is issued before the first reduction (one
// round trip instead of three), and nothing is read twice.
template <typename TD, typename TY, int NPT>
__global__ __launch_bounds__(256) void sandwich_norm_reg_kernel(const float* x, const TD* __restrict__ delta,
                                                                int64_t ld_delta, const float* __restrict__ post_w, float post_add,
                                                                float* x_out, const float* __restrict__ pre_w,
                                                                float pre_add, TY* __restrict__ y, int64_t E, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float xv[NPT], dv[NPT], pw[NPT], qw[NPT];
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int64_t c = threadIdx.x + 256 * i;
        const bool in = c < E;
        xv[i] = in ? x[row * E + c] : 0.f;
        dv[i] = (in && delta) ? Elem<TD>::ld(delta + row * ld_delta + c) : 0.f;
        pw[i] = (in && delta) ? post_w[c] + post_add : 0.f;
        qw[i] = (in && pre_w) ? pre_w[c] + pre_add : 0.f;
    }
    if (delta) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NPT; ++i) ss += dv[i] * dv[i];
        ss = block_sum(ss, red);
        const float rinv_d = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
        for (int i = 0; i < NPT; ++i) xv[i] += dv[i] * rinv_d * pw[i];
    }
    if (delta || x_out != x) {
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            const int64_t c = threadIdx.x + 256 * i;
            if (c < E) x_out[row * E + c] = xv[i];
        }
    }
    if (!pre_w) return;
    float ss2 = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) ss2 += xv[i] * xv[i];
    ss2 = block_sum(ss2, red);
    const float rinv = 1.0f / sqrtf(ss2 / (float)E + eps);
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int64_t c = threadIdx.x + 256 * i;
        if (c < E) y[row * E + c] = cvt_out<TY>(xv[i] * rinv * qw[i]);
    }
}


// The same again for E % 4 == 0 and E <= 512 * 4 * NV: 512 threads, 16-byte loads and stores (a thread owns NV groups of four
// consecutive elements).  This is the form decode-sized steps run: few rows, so the launch is a chain of round trips and the
// number of memory instructions in it is what counts.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ f32x4 ld(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
    static __device__ __forceinline__ void st(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
};
template <> struct Vec4<bf16> {
    static __device__ __forceinline__ f32x4 ld(const bf16* p) {
        bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
        return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    }
    static __device__ __forceinline__ void st(bf16* p, f32x4 v) {
        *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
    }
};
template <> struct Vec4<f16> {
    static __device__ __forceinline__ f32x4 ld(const f16* p) {
        f16x4 v = *reinterpret_cast<const f16x4*>(p);
        return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    }
    static __device__ __forceinline__ void st(f16* p, f32x4 v) {
        *reinterpret_cast<f16x4*>(p) = f16x4{(f16)v[0], (f16)v[1], (f16)v[2], (f16)v[3]};
    }
};


// four elements per thread (I % 4 == 0, rows 8- / 16-byte aligned)
template <typename T>
__global__ void glu_vec_kernel(const T* __restrict__ in, int64_t ld_in, T* __restrict__ out, int64_t ld_out, int64_t rows, int64_t I,
                               int mode, float alpha, float limit) {
    const int64_t I4 = I >> 2, n = rows * I4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / I4, i = (idx - t * I4) * 4;
        f32x4 g = Vec4<T>::ld(in + t * ld_in + i);
        f32x4 u = Vec4<T>::ld(in + t * ld_in + I + i);
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (mode == 0) {
                r[e] = g[e] / (1.f + expf(-g[e])) * u[e];
            } else {
                const float ge = fminf(g[e], limit), ue = fminf(fmaxf(u[e], -limit), limit);
                r[e] = ge / (1.f + expf(-alpha * ge)) * (ue + 1.f);
            }
        }
        Vec4<T>::st(out + t * ld_out + i, r);
    }
}

// delta may also arrive as the S fp32 split-K slabs of the GEMM that produced it ([row / 32][S][32][slab_ld], TD = float,
// `delta` then points at the slabs): their sum is taken here instead of by a reduce launch of its own.
template <typename TD, typename TY, int NV>
__global__ __launch_bounds__(512) void sandwich_norm_vec_kernel(const float* x, const TD* __restrict__ delta, int64_t ld_delta,
                                                                const float* __restrict__ post_w, float post_add, float* x_out,
                                                                const float* __restrict__ pre_w, float pre_add,
                                                                TY* __restrict__ y, int64_t E, float eps, int S) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    f32x4 xv[NV], dv[NV], pw[NV], qw[NV];
    if (S > 0) {  // slabs: ld_delta is the slab row stride
        const float* sp = reinterpret_cast<const float*>(delta) + ((row >> 5) * S * 32 + (row & 31)) * ld_delta;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
            f32x4 acc = {};
            if (c < E)
                for (int sidx = 0; sidx < S; ++sidx) acc += Vec4<float>::ld(sp + (int64_t)sidx * 32 * ld_delta + c);
            dv[i] = acc;
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        const bool in = c < E;
        xv[i] = in ? Vec4<float>::ld(x + row * E + c) : f32x4{};
        if (S == 0) dv[i] = (in && delta) ? Vec4<TD>::ld(delta + row * ld_delta + c) : f32x4{};
        pw[i] = (in && delta) ? Vec4<float>::ld(post_w + c) + post_add : f32x4{};
        qw[i] = (in && pre_w) ? Vec4<float>::ld(pre_w + c) + pre_add : f32x4{};
    }
    if (delta) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) ss += dv[i][0] * dv[i][0] + dv[i][1] * dv[i][1] + dv[i][2] * dv[i][2] + dv[i][3] * dv[i][3];
        ss = block_sum(ss, red);
        const float rinv_d = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
        for (int i = 0; i < NV; ++i) xv[i] += dv[i] * rinv_d * pw[i];
    }
    if (delta || x_out != x) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
            if (c < E) Vec4<float>::st(x_out + row * E + c, xv[i]);
        }
    }
    if (!pre_w) return;
    float ss2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) ss2 += xv[i][0] * xv[i][0] + xv[i][1] * xv[i][1] + xv[i][2] * xv[i][2] + xv[i][3] * xv[i][3];
    ss2 = block_sum(ss2, red);
    const float rinv = 1.0f / sqrtf(ss2 / (float)E + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        if (c < E) Vec4<TY>::st(y + row * E + c, xv[i] * rinv * qw[i]);
    }
}

// out[t, i] = act(gate) * up' with gate = in[t, i], up = in[t, I + i]
//   mode 0: silu(gate) * up
//   mode 1: g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha * g) * (u + 1)
template <typename T>
__global__ void glu_kernel(const T* __restrict__ in, int64_t ld_in, T* __restrict__ out, int64_t ld_out, int64_t rows, int64_t I,
                           int mode, float alpha, float limit) {
    const int64_t n = rows * I;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / I, i = idx - t * I;
        float g = Elem<T>::ld(in + t * ld_in + i);
        float u = Elem<T>::ld(in + t * ld_in + I + i);
        float r;
        if (mode == 0) {
            r = g / (1.f + expf(-g)) * u;
        } else {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
            r = g / (1.f + expf(-alpha * g)) * (u + 1.f);
        }
        out[t * ld_out + i] = cvt_out<T>(r);
    }
}

template <typename TD, typename TY>
int launch_sandwich(const float* x, const void* delta, int64_t ld_delta, const float* post_w, float post_add, float* x_out,
                    const float* pre_w, float pre_add, void* y, int64_t rows, int64_t E, float eps, hipStream_t st, int num_slabs) {
#define TGIS_SANDWICH_REG(NPT)                                                                                                  \
    hipLaunchKernelGGL((sandwich_norm_reg_kernel<TD, TY, NPT>), dim3((unsigned)rows), dim3(256), 0, st, x, (const TD*)delta, ld_delta, \
                       post_w, post_add, x_out, pre_w, pre_add, (TY*)y, E, eps)
#define TGIS_SANDWICH_VEC(NV)                                                                                                  \
    hipLaunchKernelGGL((sandwich_norm_vec_kernel<TD, TY, NV>), dim3((unsigned)rows), dim3(512), 0, st, x, (const TD*)delta, ld_delta, \
                       post_w, post_add, x_out, pre_w, pre_add, (TY*)y, E, eps, num_slabs)
    const bool vec_ok = E % 4 == 0 && (!delta || ld_delta % 4 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)x_out % 16 == 0) &&
                        ((uintptr_t)delta % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)post_w % 16 == 0) &&
                        ((uintptr_t)pre_w % 16 == 0);
    if (num_slabs > 0 && !(vec_ok && E <= 512 * 16)) return -1;  // slabs are taken by the 16-byte form only
    if (vec_ok && E <= 512 * 4)
        TGIS_SANDWICH_VEC(1);
    else if (vec_ok && E <= 512 * 8)
        TGIS_SANDWICH_VEC(2);
    else if (vec_ok && E <= 512 * 16)
        TGIS_SANDWICH_VEC(4);
    else if (E <= 256 * 4)
        TGIS_SANDWICH_REG(4);
    else if (E <= 256 * 8)
        TGIS_SANDWICH_REG(8);
    else if (E <= 256 * 16)
        TGIS_SANDWICH_REG(16);
    else if (E <= 256 * 32)
        TGIS_SANDWICH_REG(32);
    else
        hipLaunchKernelGGL((sandwich_norm_kernel<TD, TY>), dim3((unsigned)rows), dim3(256), 0, st, x, (const TD*)delta, ld_delta,
                           post_w, post_add, x_out, pre_w, pre_add, (TY*)y, E, eps);
#undef TGIS_SANDWICH_REG
#undef TGIS_SANDWICH_VEC
    return 0;
}

template <typename TD>
int dispatch_y(int y_dtype, const float* x, const void* delta, int64_t ld_delta, const float* post_w, float post_add,
               float* x_out, const float* pre_w, float pre_add, void* y, int64_t rows, int64_t E, float eps, hipStream_t st,
               int num_slabs = 0) {
    switch (y_dtype) {
        case TGIS_F16: return launch_sandwich<TD, f16>(x, delta, ld_delta, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
        case TGIS_BF16: return launch_sandwich<TD, bf16>(x, delta, ld_delta, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
        default: return launch_sandwich<TD, float>(x, delta, ld_delta, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
    }
}

}  // namespace

static bool dtype3(int d) { return d == TGIS_F16 || d == TGIS_BF16 || d == TGIS_F32; }

extern "C" int tgis_embedding_scaled_f32(const int64_t* ids, const void* table, float* out, int64_t T, int64_t E, int64_t vocab,
                                         float scale, int dtype, void* stream) {
    TGIS_CHECK_ARG(ids && table && out && E > 0 && vocab > 0, "tgis_embedding_scaled_f32: bad arguments");
    TGIS_CHECK_ARG(dtype3(dtype), "tgis_embedding_scaled_f32: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(embedding_scaled_kernel<f16>, dim3((unsigned)T), dim3(256), 0, st, ids, (const f16*)table, out, E, vocab, scale);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(embedding_scaled_kernel<bf16>, dim3((unsigned)T), dim3(256), 0, st, ids, (const bf16*)table, out, E, vocab, scale);
    else
        hipLaunchKernelGGL(embedding_scaled_kernel<float>, dim3((unsigned)T), dim3(256), 0, st, ids, (const float*)table, out, E, vocab, scale);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_sandwich_norm_f32(const float* x, const void* delta, int64_t ld_delta, int delta_dtype, const float* post_w,
                                      float post_add, float* x_out, const float* pre_w, float pre_add, void* y, int y_dtype,
                                      int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && x_out && E > 0 && rows >= 0, "tgis_sandwich_norm_f32: bad arguments");
    TGIS_CHECK_ARG(!delta || (post_w && ld_delta >= E && dtype3(delta_dtype)), "tgis_sandwich_norm_f32: delta needs its gain, a row stride and a dtype");
    TGIS_CHECK_ARG(!pre_w || (y && dtype3(y_dtype)), "tgis_sandwich_norm_f32: the normed output needs a buffer and a dtype");
    TGIS_CHECK_ARG(delta || pre_w || x_out != x, "tgis_sandwich_norm_f32: nothing to do");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const int dd = delta ? delta_dtype : TGIS_F32;
    if (dd == TGIS_F16)
        dispatch_y<f16>(y_dtype, x, delta, ld_delta, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st);
    else if (dd == TGIS_BF16)
        dispatch_y<bf16>(y_dtype, x, delta, ld_delta, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st);
    else
        dispatch_y<float>(y_dtype, x, delta, ld_delta, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_glu(const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int64_t I, int mode, float alpha,
                        float limit, int dtype, void* stream) {
    TGIS_CHECK_ARG(in && out && I > 0 && ld_in >= 2 * I && ld_out >= I, "tgis_glu: bad arguments");
    TGIS_CHECK_ARG(mode == 0 || mode == 1, "tgis_glu: mode 0 (silu(gate) * up) or 1 (clamped, sigmoid(alpha g), up + 1)");
    TGIS_CHECK_ARG(dtype3(dtype), "tgis_glu: bad dtype");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    const int esz = dtype == TGIS_F32 ? 4 : 2;
    const bool vec = I % 4 == 0 && ld_in % 4 == 0 && ld_out % 4 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                     (I * esz) % 8 == 0;
    const int64_t n = vec ? rows * (I / 4) : rows * I;
    dim3 grid((unsigned)(cdiv64(n, 256) < 16384 ? cdiv64(n, 256) : 16384));
#define TGIS_GLU(KERNEL, TT) \
    hipLaunchKernelGGL(KERNEL<TT>, grid, dim3(256), 0, st, (const TT*)in, ld_in, (TT*)out, ld_out, rows, I, mode, alpha, limit)
    if (dtype == TGIS_F16) {
        if (vec) TGIS_GLU(glu_vec_kernel, f16); else TGIS_GLU(glu_kernel, f16);
    } else if (dtype == TGIS_BF16) {
        if (vec) TGIS_GLU(glu_vec_kernel, bf16); else TGIS_GLU(glu_kernel, bf16);
    } else {
        if (vec) TGIS_GLU(glu_vec_kernel, float); else TGIS_GLU(glu_kernel, float);
    }
#undef TGIS_GLU
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_sandwich_norm_f32_partial(const float* x, const float* slabs, int num_slabs, int64_t slab_ld, const float* post_w,
                                              float post_add, float* x_out, const float* pre_w, float pre_add, void* y, int y_dtype,
                                              int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && x_out && slabs && post_w && E > 0 && rows >= 0, "tgis_sandwich_norm_f32_partial: bad arguments");
    TGIS_CHECK_ARG(num_slabs >= 1 && slab_ld >= E && slab_ld % 4 == 0, "tgis_sandwich_norm_f32_partial: bad slab geometry");
    TGIS_CHECK_ARG(!pre_w || (y && dtype3(y_dtype)), "tgis_sandwich_norm_f32_partial: the normed output needs a buffer and a dtype");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const int rc = dispatch_y<float>(y_dtype, x, slabs, slab_ld, post_w, post_add, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
    TGIS_CHECK_ARG(rc == 0, "tgis_sandwich_norm_f32_partial: needs E %% 4 == 0, E <= 8192 and 16-byte aligned operands");
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
