// Linear-recurrence ("wkv", RWKV-style) time mixing with state slots:
//   token shift   mix_s[t] = h[t] + (h[t-1] - h[t]) * mu_s           (h[-1] of a step's first token comes from the slot)
//   decay         log w[t] = -exp(w0 + W2 tanh(a[t]))                 (a = the rank-reduced projection of mix_w, done by a GEMM)
//   recurrence    o[t] = (S + diag(u) k[t] v[t]^T)^T r[t];   S <- diag(w[t]) S + k[t] v[t]^T      per head, S in fp32
//   output        o / rms(o) per head, * gain * silu(gate)
// State per slot: S[head][key channel][value channel] (fp32) and the last token's mixer input (fp32).  A sequence whose
// step starts at position 0 starts from zeros whatever its slot held before: slots need no clearing when they change hands.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }

__device__ __forceinline__ int seq_of_token(const int32_t* __restrict__ cu_q, int B, int t) {
    int lo = 0, hi = B;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

// one workgroup per token; out[s][t][c], s < NM
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(const float* __restrict__ h, const float* __restrict__ shift_state,
                                                              const int32_t* __restrict__ state_slots, const int32_t* __restrict__ cu_q,
                                                              const int32_t* __restrict__ positions, int B, const float* __restrict__ mu,
                                                              int NM, T* __restrict__ out, int64_t Ttot, int64_t W) {
    const int t = blockIdx.x;
    const int b = seq_of_token(cu_q, B, t);
    const bool first = t == cu_q[b];
    const bool fresh = first && positions[t] == 0;
    const float* prev = first ? shift_state + (int64_t)state_slots[b] * W : h + (int64_t)(t - 1) * W;
    const float* cur = h + (int64_t)t * W;
    // grid (token, 256-column block): one element per thread, so that a decode step's few tokens still fill the chip
    const int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= W) return;
    const float x = cur[c];
    const float d = (fresh ? 0.f : prev[c]) - x;
    for (int s = 0; s < NM; ++s) out[((int64_t)s * Ttot + t) * W + c] = (T)(x + d * mu[(int64_t)s * W + c]);
}

// grid (token, 256-channel block): logw[t][c] = -exp(w0[c] + sum_r tanh(a[t][r]) * w2t[r][c])
template <typename T>
__global__ __launch_bounds__(256) void wkv_decay_kernel(const T* __restrict__ a, int64_t ld_a, const float* __restrict__ w2t,
                                                        const float* __restrict__ w0, float* __restrict__ logw, int R, int64_t C) {
    extern __shared__ float th[];
    const int64_t t = blockIdx.x;
    for (int r = threadIdx.x; r < R; r += blockDim.x) th[r] = tanhf(ldf(a + t * ld_a + r));
    __syncthreads();
    const int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    float z = w0[c];
#pragma unroll 8
    for (int r = 0; r < R; ++r) z += th[r] * w2t[(int64_t)r * C + c];
    logw[t * C + c] = -expf(z);
}

// One workgroup per (sequence, head) = four thread groups: thread (q, j) owns value channel j and keeps the rows
// i in [q DQ, (q + 1) DQ) of column j of S in registers (rows of S evolve independently of each other, so the four groups
// never have to meet inside a token: each leaves its part of o in LDS and the parts are added once per chunk).  Tokens are
// staged through LDS CH at a time; all threads of a wave read the same r / k / w element at the same time (LDS broadcast).
// The next chunk's r, k, v, gate and log-decay are fetched into registers while the current one is computed.
constexpr int CH = 16;
constexpr int IS = 4;  // row groups

template <typename T, int DMAX>
__global__ __launch_bounds__((DMAX < 64 ? 64 : DMAX) * IS) void wkv_scan_kernel(
    const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, const T* __restrict__ gate, int64_t ld,
    const float* __restrict__ logw, const float* __restrict__ u, const float* __restrict__ gain, float* __restrict__ state,
    float* __restrict__ shift_state, const float* __restrict__ h, int64_t W, const int32_t* __restrict__ state_slots,
    const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions, T* __restrict__ out, int64_t ld_out, int H, int d,
    float eps) {
    constexpr int NJ = DMAX < 64 ? 64 : DMAX;  // threads per row group (whole waves)
    constexpr int NT = NJ * IS;
    constexpr int DQ = DMAX / IS;
    constexpr int PER = (CH * DMAX + NT - 1) / NT;
    __shared__ float rr[CH][DMAX], kk[CH][DMAX], ww[CH][DMAX], vv[CH][DMAX], gg[CH][DMAX], oo[IS][CH][DMAX], us[DMAX];
    const int b = blockIdx.x, head = blockIdx.y;
    const int tid = threadIdx.x;
    const int q = tid / NJ, j = tid % NJ;
    const int t0 = cu_q[b], t1 = cu_q[b + 1];
    if (t1 <= t0) return;
    const int64_t slot = state_slots[b];
    const bool fresh = positions[t0] == 0;
    float* Sg = state + ((slot * H + head) * d) * (int64_t)d;  // [i][j]
    float S[DQ];
#pragma unroll
    for (int ii = 0; ii < DQ; ++ii) {
        const int i = q * DQ + ii;
        S[ii] = (!fresh && i < d && j < d) ? Sg[(int64_t)i * d + j] : 0.f;
    }
    if (tid < DMAX) us[tid] = tid < d ? u[head * d + tid] : 0.f;
    const int64_t col0 = (int64_t)head * d;
    const int64_t C = (int64_t)H * d;
    float pr[PER], pk[PER], pv[PER], pg[PER], pw[PER];
    auto fetch = [&](int tc) {
        const int n = min(CH, t1 - tc);
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int idx = tid + e * NT, tt = idx / DMAX, i = idx % DMAX;
            const bool ok = tt < n && i < d;
            const int64_t at = (int64_t)(tc + tt) * ld + col0 + i;
            pr[e] = ok ? ldf(r + at) : 0.f;
            pk[e] = ok ? ldf(k + at) : 0.f;
            pv[e] = ok ? ldf(v + at) : 0.f;
            pg[e] = ok ? ldf(gate + at) : 0.f;
            pw[e] = ok ? logw[(int64_t)(tc + tt) * C + col0 + i] : 0.f;
        }
    };
    fetch(t0);
    for (int tc = t0; tc < t1; tc += CH) {
        const int n = min(CH, t1 - tc);
        __syncthreads();  // the previous chunk is consumed
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int idx = tid + e * NT, tt = idx / DMAX, i = idx % DMAX;
            if (tt < CH) {
                rr[tt][i] = pr[e];
                kk[tt][i] = pk[e];
                vv[tt][i] = pv[e];
                gg[tt][i] = pg[e];
                ww[tt][i] = expf(pw[e]);
            }
        }
        __syncthreads();
        if (tc + CH < t1) fetch(tc + CH);
        const int jj = j < DMAX ? j : 0;
        for (int tt = 0; tt < n; ++tt) {
            const float vj = vv[tt][jj];
            float a = 0.f, bonus = 0.f;
#pragma unroll
            for (int ii = 0; ii < DQ; ++ii) {
                const int i = q * DQ + ii;
                const float ri = rr[tt][i], ki = kk[tt][i];
                a += ri * S[ii];
                bonus += ri * us[i] * ki;
                S[ii] = ww[tt][i] * S[ii] + ki * vj;
            }
            if (j < DMAX) oo[q][tt][j] = a + bonus * vj;
        }
        __syncthreads();
        // the row groups' parts are added; per-head unit norm, gain, gate: one wave per token
        const int wave = tid >> 6, lane = tid & 63, nw = NT >> 6;
        for (int tt = wave; tt < n; tt += nw) {
            float ov[(DMAX + 63) / 64];
            float ss = 0.f;
#pragma unroll
            for (int cc = 0; cc < (DMAX + 63) / 64; ++cc) {
                const int c = lane + 64 * cc;
                float o = 0.f;
                if (c < d) {
#pragma unroll
                    for (int g4 = 0; g4 < IS; ++g4) o += oo[g4][tt][c];
                }
                ov[cc] = o;
                ss += o * o;
            }
            ss = wave_sum(ss);
            const float rinv = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
            for (int cc = 0; cc < (DMAX + 63) / 64; ++cc) {
                const int c = lane + 64 * cc;
                if (c < d) {
                    const float gt = gg[tt][c];
                    out[(int64_t)(tc + tt) * ld_out + col0 + c] = (T)(ov[cc] * rinv * gain[col0 + c] * (gt / (1.f + expf(-gt))));
                }
            }
        }
    }
    if (j < d) {
#pragma unroll
        for (int ii = 0; ii < DQ; ++ii) {
            const int i = q * DQ + ii;
            if (i < d) Sg[(int64_t)i * d + j] = S[ii];
        }
    }
    if (head == 0) {
        const float* last = h + (int64_t)(t1 - 1) * W;
        float* dst = shift_state + slot * W;
        for (int64_t c = tid; c < W; c += NT) dst[c] = last[c];
    }
}

template <typename T>
int launch_scan(const void* r, const void* k, const void* v, const void* gate, int64_t ld, const float* logw, const float* u,
                const float* gain, float* state, float* shift_state, const float* h, int64_t W, const int32_t* slots,
                const int32_t* cu_q, const int32_t* positions, void* out, int64_t ld_out, int B, int H, int d, float eps,
                hipStream_t st) {
#define TGIS_WKV_LAUNCH(DM)                                                                                               \
    hipLaunchKernelGGL((wkv_scan_kernel<T, DM>), dim3((unsigned)B, (unsigned)H), dim3((DM < 64 ? 64 : DM) * IS), 0, st, (const T*)r, \
                       (const T*)k, (const T*)v, (const T*)gate, ld, logw, u, gain, state, shift_state, h, W, slots, cu_q,    \
                       positions, (T*)out, ld_out, H, d, eps)
    if (d <= 32)
        TGIS_WKV_LAUNCH(32);
    else if (d <= 64)
        TGIS_WKV_LAUNCH(64);
    else
        TGIS_WKV_LAUNCH(128);
#undef TGIS_WKV_LAUNCH
    return 0;
}

}  // namespace

static bool dtype3(int d) { return d == TGIS_F16 || d == TGIS_BF16 || d == TGIS_F32; }

extern "C" int tgis_token_shift_mix(const float* h, const float* shift_state, const int32_t* state_slots, const int32_t* cu_seqlens_q,
                                    const int32_t* positions, int64_t B, const float* mu, int num_mixes, void* out, int64_t T,
                                    int64_t W, int dtype, void* stream) {
    TGIS_CHECK_ARG(h && shift_state && state_slots && cu_seqlens_q && positions && mu && out, "tgis_token_shift_mix: null tensor");
    TGIS_CHECK_ARG(B >= 1 && num_mixes >= 1 && W >= 1 && dtype3(dtype), "tgis_token_shift_mix: bad arguments");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(token_shift_mix_kernel<f16>, dim3((unsigned)T, (unsigned)cdiv64(W, 256)), dim3(256), 0, st, h, shift_state, state_slots, cu_seqlens_q, positions, (int)B, mu, num_mixes, (f16*)out, T, W);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(token_shift_mix_kernel<bf16>, dim3((unsigned)T, (unsigned)cdiv64(W, 256)), dim3(256), 0, st, h, shift_state, state_slots, cu_seqlens_q, positions, (int)B, mu, num_mixes, (bf16*)out, T, W);
    else
        hipLaunchKernelGGL(token_shift_mix_kernel<float>, dim3((unsigned)T, (unsigned)cdiv64(W, 256)), dim3(256), 0, st, h, shift_state, state_slots, cu_seqlens_q, positions, (int)B, mu, num_mixes, (float*)out, T, W);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_wkv_decay(const void* a, int64_t ld_a, const float* w2t, const float* w0, float* logw, int64_t T, int rank,
                              int64_t C, int dtype, void* stream) {
    TGIS_CHECK_ARG(a && w2t && w0 && logw && rank >= 1 && rank <= 8192 && C >= 1 && C <= 65535 * 256 && ld_a >= rank && dtype3(dtype), "tgis_wkv_decay: bad arguments");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = (size_t)rank * sizeof(float);
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(wkv_decay_kernel<f16>, dim3((unsigned)T, (unsigned)cdiv64(C, 256)), dim3(256), lds, st, (const f16*)a, ld_a, w2t, w0, logw, rank, C);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(wkv_decay_kernel<bf16>, dim3((unsigned)T, (unsigned)cdiv64(C, 256)), dim3(256), lds, st, (const bf16*)a, ld_a, w2t, w0, logw, rank, C);
    else
        hipLaunchKernelGGL(wkv_decay_kernel<float>, dim3((unsigned)T, (unsigned)cdiv64(C, 256)), dim3(256), lds, st, (const float*)a, ld_a, w2t, w0, logw, rank, C);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_wkv_scan(const void* r, const void* k, const void* v, const void* gate, int64_t ld, const float* logw,
                             const float* u, const float* gain, float* state, float* shift_state, const float* h, int64_t W,
                             const int32_t* state_slots, const int32_t* cu_seqlens_q, const int32_t* positions, void* out,
                             int64_t ld_out, int64_t B, int H, int d, float eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(r && k && v && gate && logw && u && gain && state && shift_state && h && state_slots && cu_seqlens_q &&
                       positions && out,
                   "tgis_wkv_scan: null tensor");
    TGIS_CHECK_ARG(B >= 1 && H >= 1 && d >= 1 && d <= 128, "tgis_wkv_scan: head width %d (1 .. 128 supported)", d);
    TGIS_CHECK_ARG(ld >= (int64_t)H * d && ld_out >= (int64_t)H * d && W >= 1 && dtype3(dtype), "tgis_wkv_scan: bad strides or dtype");
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    if (dtype == TGIS_F16)
        launch_scan<f16>(r, k, v, gate, ld, logw, u, gain, state, shift_state, h, W, state_slots, cu_seqlens_q, positions, out, ld_out, (int)B, H, d, eps, st);
    else if (dtype == TGIS_BF16)
        launch_scan<bf16>(r, k, v, gate, ld, logw, u, gain, state, shift_state, h, W, state_slots, cu_seqlens_q, positions, out, ld_out, (int)B, H, d, eps, st);
    else
        launch_scan<float>(r, k, v, gate, ld, logw, u, gain, state, shift_state, h, W, state_slots, cu_seqlens_q, positions, out, ld_out, (int)B, H, d, eps, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
