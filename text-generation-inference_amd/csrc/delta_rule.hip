// Gated delta-rule time mixing with one decay per head and key channel, on state slots:
//   short convolution   c[t] = silu(sum_j w[ch][j] x[t - (taps - 1 - j)][ch])     per channel of q | k | v, causal, no bias
//   unit vectors        q <- q / sqrt(|q|^2 + unit_eps) * q_scale,  k <- k / sqrt(|k|^2 + unit_eps)      per head
//   gates               beta = sigmoid(b),   g = exp(-exp(A_log[head]) * softplus(a + dt_bias))            g per key channel
//   recurrence          S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                  S [dk][dv], fp32
//   output              o / rms(o) per head * gain[dv] * sigmoid(gate)
// State per slot: S of every head (fp32, in the scan kernel's own thread order, see delta_scan_kernel) and the last taps - 1
// inputs of the convolution (fp32, [taps - 1][channels]).  A sequence whose step starts at position 0 starts from zeros
// whatever its slot held before: slots need no clearing when they change hands.
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

__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// grid (token, 256-channel block): the step's own tokens are read from x, the ones before it from the slot's tail
template <typename T>
__global__ __launch_bounds__(256) void short_conv_silu_kernel(const T* __restrict__ x, int64_t ld_x, const float* __restrict__ w,
                                                              const float* __restrict__ tail, const int32_t* __restrict__ state_slots,
                                                              const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                                              int B, float* __restrict__ out, int64_t C, int taps) {
    const int t = blockIdx.x;
    const int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int b = seq_of_token(cu_q, B, t);
    const int t0 = cu_q[b];
    const bool fresh = positions[t0] == 0;
    const float* tl = tail + (int64_t)state_slots[b] * (taps - 1) * C;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int i = (t - t0) - (taps - 1 - j);  // index among the step's tokens of this sequence
        float v;
        if (i >= 0)
            v = ldf(x + (int64_t)(t0 + i) * ld_x + c);
        else
            v = fresh ? 0.f : tl[(int64_t)(taps - 1 + i) * C + c];
        acc += w[c * taps + j] * v;
    }
    out[(int64_t)t * C + c] = acc / (1.f + expf(-acc));
}

// The same, four neighbouring channels per thread (C % 4 == 0, rows 8- / 16-byte aligned): one 8- or 16-byte load per tap,
// one 16-byte store — the form long steps run, where the launch is bound by its traffic.
template <typename T> struct Ld4;
template <> struct Ld4<float> {
    static __device__ __forceinline__ f32x4 ld(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
};
template <> struct Ld4<bf16> {
    static __device__ __forceinline__ f32x4 ld(const bf16* p) {
        bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
        return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    }
};
template <> struct Ld4<f16> {
    static __device__ __forceinline__ f32x4 ld(const f16* p) {
        f16x4 v = *reinterpret_cast<const f16x4*>(p);
        return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    }
};

template <typename T>
__global__ __launch_bounds__(256) void short_conv_silu_vec_kernel(const T* __restrict__ x, int64_t ld_x, const float* __restrict__ w,
                                                                  const float* __restrict__ tail, const int32_t* __restrict__ state_slots,
                                                                  const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                                                  int B, float* __restrict__ out, int64_t C, int taps) {
    const int t = blockIdx.x;
    const int64_t c = ((int64_t)blockIdx.y * blockDim.x + threadIdx.x) * 4;
    if (c >= C) return;
    const int b = seq_of_token(cu_q, B, t);
    const int t0 = cu_q[b];
    const bool fresh = positions[t0] == 0;
    const float* tl = tail + (int64_t)state_slots[b] * (taps - 1) * C;
    f32x4 acc = {};
    for (int j = 0; j < taps; ++j) {
        const int i = (t - t0) - (taps - 1 - j);
        f32x4 v = {};
        if (i >= 0)
            v = Ld4<T>::ld(x + (int64_t)(t0 + i) * ld_x + c);
        else if (!fresh)
            v = *reinterpret_cast<const f32x4*>(tl + (int64_t)(taps - 1 + i) * C + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += w[(c + e) * taps + j] * v[e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = acc[e] / (1.f + expf(-acc[e]));
    *reinterpret_cast<f32x4*>(out + (int64_t)t * C + c) = acc;
}

// Long steps: a thread walks TB consecutive tokens for its four channels with the last TAPS - 1 inputs in registers — one
// load per token instead of TAPS, and the walk through cu_q / positions / slots once per TB tokens.  A run may cross into
// the next sequence of the step: the window is then filled again from that sequence's tail.
constexpr int TB = 8;
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void short_conv_silu_run_kernel(const T* __restrict__ x, int64_t ld_x, const float* __restrict__ w,
                                                                  const float* __restrict__ tail, const int32_t* __restrict__ state_slots,
                                                                  const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                                                  int B, float* __restrict__ out, int64_t Ttot, int64_t C) {
    const int64_t c = ((int64_t)blockIdx.y * blockDim.x + threadIdx.x) * 4;
    if (c >= C) return;
    const int tb = blockIdx.x * TB;
    f32x4 wt[TAPS];
#pragma unroll
    for (int j = 0; j < TAPS; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) wt[j][e] = w[(c + e) * TAPS + j];
    int b = seq_of_token(cu_q, B, tb);
    int t0 = cu_q[b], t1 = cu_q[b + 1];
    f32x4 win[TAPS - 1];
    auto fill = [&](int t) {  // the TAPS - 1 inputs before token t of sequence b
        const bool fresh = positions[t0] == 0;
        const float* tl = tail + (int64_t)state_slots[b] * (TAPS - 1) * C;
#pragma unroll
        for (int j = 0; j < TAPS - 1; ++j) {
            const int i = (t - t0) - (TAPS - 1 - j);
            if (i >= 0)
                win[j] = Ld4<T>::ld(x + (int64_t)(t0 + i) * ld_x + c);
            else if (!fresh)
                win[j] = *reinterpret_cast<const f32x4*>(tl + (int64_t)(TAPS - 1 + i) * C + c);
            else
                win[j] = f32x4{};
        }
    };
    fill(tb);
    for (int tt = 0; tt < TB; ++tt) {
        const int t = tb + tt;
        if (t >= Ttot) break;
        if (t >= t1) {
            while (t >= cu_q[b + 1]) ++b;
            t0 = cu_q[b];
            t1 = cu_q[b + 1];
            fill(t);
        }
        const f32x4 cur = Ld4<T>::ld(x + (int64_t)t * ld_x + c);
        f32x4 acc = {};
        // the same order of sums as the per-token kernels: oldest tap first
#pragma unroll
        for (int j = 0; j < TAPS - 1; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += wt[j][e] * win[j][e];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += wt[TAPS - 1][e] * cur[e];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = acc[e] / (1.f + expf(-acc[e]));
        *reinterpret_cast<f32x4*>(out + (int64_t)t * C + c) = acc;
#pragma unroll
        for (int j = 0; j + 1 < TAPS - 1; ++j) win[j] = win[j + 1];
        win[TAPS - 2] = cur;
    }
}

constexpr int CH = 16;  // tokens per LDS stage
constexpr int RS = 4;   // lanes that share a column of S (row groups)

// sum over the four neighbouring lanes of a quad, by data-parallel-primitive moves (no trip through LDS)
__device__ __forceinline__ float quad_sum(float v) {
    static_assert(RS == 4, "the row groups of a column are one quad");
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));  // lane ^ 1
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));  // lane ^ 2
    return v;
}

// One workgroup per (sequence, value head).  Thread tid = j * RS + r owns value channel j and keeps the rows
// i in [r DQ, (r + 1) DQ) of column j of S in registers; the RS lanes of a column are neighbours, so the two sums over the
// rows (S^T k and S^T q) meet by two lane exchanges per token and nothing else crosses threads inside a token:
//     s_i = g_i S_i;   kS = sum s_i k_i;   qS = sum s_i q_i;   u = beta (v_j - kS);   S_i = s_i + k_i u;   o_j = qS + u (k . q)
// Tokens are staged through LDS CH at a time (q, k unit-normed there, the decay and beta evaluated there); a thread reads its
// DQ rows of q / k / g with 16-byte LDS loads (row groups are 16 bytes apart in bank space).  The next stage's operands are
// fetched into registers while the current one is computed.
// State layout: state[slot][head][ii][tid] with row i = r DQ + ii — the kernel's own order, so that loading and storing the
// state (all a decode step does, in bytes) are contiguous 256-byte runs per wave.
template <typename T, int DK, int DVP>
__global__ __launch_bounds__(DVP * RS) void delta_scan_kernel(
    const float* __restrict__ conv, int64_t C, const T* __restrict__ a, int64_t ld_a, const T* __restrict__ bproj, int64_t ld_b,
    const T* __restrict__ gate, int64_t ld_g, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
    const float* __restrict__ gain, float* __restrict__ state, int64_t head_floats, float* __restrict__ tail, const T* __restrict__ proj,
    int64_t ld_p, const int32_t* __restrict__ state_slots, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
    T* __restrict__ out, int64_t ld_out, int H, int G, int dk, int dv, int taps, float eps, float unit_eps, float q_scale) {
    constexpr int DQ = DK / RS;
    constexpr int ROW = DK + RS * 4;  // a token's q / k / g row in LDS: row group r starts at r (DQ + 4)
    constexpr int NT = DVP * RS;
    constexpr int PERK = (CH * DK + NT - 1) / NT;  // staged q / k / a elements per thread
    constexpr int PERV = CH / RS;                  // staged v / gate elements per thread (CH DVP / NT)
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* qs = smem;                  // [CH][ROW]
    float* ks = qs + CH * ROW;         // [CH][ROW]
    float* gs = ks + CH * ROW;         // [CH][ROW]
    float* vs = gs + CH * ROW;         // [CH][DVP]
    float* gt = vs + CH * DVP;         // [CH][DVP] raw output gate
    float* oo = gt + CH * DVP;         // [CH][DVP]
    float* bt = oo + CH * DVP;         // [CH] beta
    float* kq = bt + CH;               // [CH] k . q
    const int b = blockIdx.x, head = blockIdx.y;
    const int tid = threadIdx.x, r = tid % RS, j = tid / RS;
    const int t0 = cu_q[b], t1 = cu_q[b + 1];
    if (t1 <= t0) return;
    const int64_t slot = state_slots[b];
    const bool fresh = positions[t0] == 0;
    const int g = head / (H / G);
    float* Sg = state + (slot * H + head) * head_floats;
    float S[DQ];
#pragma unroll
    for (int ii = 0; ii < DQ; ++ii) S[ii] = fresh ? 0.f : Sg[(int64_t)ii * NT + tid];
    const float a_rate = -expf(A_log[head]);
    const int64_t qc = (int64_t)g * dk, kc = (int64_t)G * dk + (int64_t)g * dk, vc = (int64_t)2 * G * dk + (int64_t)head * dv;
    // staging slots of this thread: element e of the [CH][DK] operands and of the [CH][DVP] ones
    float pq[PERK], pk[PERK], pa[PERK], pv[PERV], pg[PERV];
    float pb = 0.f;
    auto fetch = [&](int tc) {
        const int n = min(CH, t1 - tc);
#pragma unroll
        for (int e = 0; e < PERK; ++e) {
            const int idx = tid + e * NT, tt = idx / DK, i = idx % DK;
            const bool ok = tt < n && i < dk;
            const int64_t row = (int64_t)(tc + tt);
            pq[e] = ok ? conv[row * C + qc + i] : 0.f;
            pk[e] = ok ? conv[row * C + kc + i] : 0.f;
            pa[e] = ok ? ldf(a + row * ld_a + (int64_t)head * dk + i) : 0.f;
        }
#pragma unroll
        for (int e = 0; e < PERV; ++e) {
            const int idx = tid + e * NT, tt = idx / DVP, c = idx % DVP;
            const bool ok = tt < n && c < dv;
            const int64_t row = (int64_t)(tc + tt);
            pv[e] = ok ? conv[row * C + vc + c] : 0.f;
            pg[e] = ok ? ldf(gate + row * ld_g + (int64_t)head * dv + c) : 0.f;
        }
        if (tid < CH) pb = tid < n ? ldf(bproj + (int64_t)(tc + tid) * ld_b + head) : 0.f;
    };
    fetch(t0);
    for (int tc = t0; tc < t1; tc += CH) {
        const int n = min(CH, t1 - tc);
        __syncthreads();  // the previous stage is consumed
#pragma unroll
        for (int e = 0; e < PERK; ++e) {
            const int idx = tid + e * NT, tt = idx / DK, i = idx % DK;
            if (tt < CH) {
                const int at = tt * ROW + i + (i / DQ) * 4;
                qs[at] = pq[e];
                ks[at] = pk[e];
                // rows past dk: g = 1, k = q = 0 leave the padded part of S at zero
                gs[at] = i < dk ? expf(a_rate * softplus_f32(pa[e] + dt_bias[head * dk + i])) : 1.f;
            }
        }
#pragma unroll
        for (int e = 0; e < PERV; ++e) {
            const int idx = tid + e * NT, tt = idx / DVP, c = idx % DVP;
            vs[tt * DVP + c] = pv[e];
            gt[tt * DVP + c] = pg[e];
        }
        if (tid < CH) bt[tid] = 1.f / (1.f + expf(-pb));
        __syncthreads();
        if (tc + CH < t1) fetch(tc + CH);
        // unit vectors and k . q: sixteen lanes per token (four tokens per wave at once), DK / 16 channels per lane, the
        // sums meet by four lane exchanges — all tokens of the stage go through those exchanges together
        for (int idx = tid; idx < CH * 16; idx += NT) {
            const int tt = idx >> 4, seg = idx & 15;
            constexpr int PER = DK / 16;
            float sq = 0.f, sk = 0.f, dot = 0.f;
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const int i = seg * PER + e;
                const int at = tt * ROW + i + (i / DQ) * 4;
                const float qv = qs[at], kv = ks[at];
                sq += qv * qv;
                sk += kv * kv;
                dot += qv * kv;
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) {
                sq += __shfl_xor(sq, o, 64);
                sk += __shfl_xor(sk, o, 64);
                dot += __shfl_xor(dot, o, 64);
            }
            const float rq = q_scale / sqrtf(sq + unit_eps), rk = 1.0f / sqrtf(sk + unit_eps);
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const int i = seg * PER + e;
                const int at = tt * ROW + i + (i / DQ) * 4;
                qs[at] *= rq;
                ks[at] *= rk;
            }
            if (seg == 0) kq[tt] = dot * rq * rk;
        }
        __syncthreads();
        const int base = r * (DQ + 4);
        for (int tt = 0; tt < n; ++tt) {
            const float* qr = qs + tt * ROW + base;
            const float* kr = ks + tt * ROW + base;
            const float* gr = gs + tt * ROW + base;
            constexpr bool KEEP_K = DQ <= 32;  // k stays in registers for the second pass; wide heads read it again
            float kk[KEEP_K ? DQ : 1];
            float kS = 0.f, qS = 0.f;
#pragma unroll
            for (int i4 = 0; i4 < DQ; i4 += 4) {
                const f32x4 g4 = *reinterpret_cast<const f32x4*>(gr + i4);
                const f32x4 k4 = *reinterpret_cast<const f32x4*>(kr + i4);
                const f32x4 q4 = *reinterpret_cast<const f32x4*>(qr + i4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float s = S[i4 + e] * g4[e];
                    S[i4 + e] = s;
                    if (KEEP_K) kk[i4 + e] = k4[e];
                    kS += s * k4[e];
                    qS += s * q4[e];
                }
            }
            kS = quad_sum(kS);
            qS = quad_sum(qS);
            const float u = bt[tt] * (vs[tt * DVP + j] - kS);
            if (KEEP_K) {
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) S[ii] += kk[ii] * u;
            } else {
#pragma unroll
                for (int i4 = 0; i4 < DQ; i4 += 4) {
                    const f32x4 k4 = *reinterpret_cast<const f32x4*>(kr + i4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) S[i4 + e] += k4[e] * u;
                }
            }
            if (r == 0) oo[tt * DVP + j] = qS + u * kq[tt];
        }
        __syncthreads();
        // per-head unit RMS, gain, output gate: sixteen lanes per token again
        for (int idx = tid; idx < CH * 16; idx += NT) {
            const int tt = idx >> 4, seg = idx & 15;
            float ss = 0.f;
            for (int c = seg; c < dv; c += 16) {
                const float o = oo[tt * DVP + c];
                ss += o * o;
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) ss += __shfl_xor(ss, o, 64);
            const float rinv = 1.0f / sqrtf(ss / (float)dv + eps);
            if (tt < n)
                for (int c = seg; c < dv; c += 16)
                    out[(int64_t)(tc + tt) * ld_out + (int64_t)head * dv + c] =
                        (T)(oo[tt * DVP + c] * rinv * gain[c] / (1.f + expf(-gt[tt * DVP + c])));
        }
    }
#pragma unroll
    for (int ii = 0; ii < DQ; ++ii) Sg[(int64_t)ii * NT + tid] = S[ii];
    // the convolution's memory: the last taps - 1 inputs of this head's channels (q / k channels by the first head of a group)
    const int n_all = t1 - t0;
    float* tl = tail + slot * (int64_t)(taps - 1) * C;
    const int nch = dv + ((head % (H / G)) == 0 ? 2 * dk : 0);
    for (int e = tid; e < nch; e += NT) {
        const int64_t c = e < dv ? vc + e : (e - dv < dk ? qc + (e - dv) : kc + (e - dv - dk));
        float keep[8];
        for (int rr = 0; rr < taps - 1; ++rr) {
            const int i = n_all - (taps - 1) + rr;
            float v;
            if (i >= 0)
                v = ldf(proj + (int64_t)(t0 + i) * ld_p + c);
            else
                v = fresh ? 0.f : tl[(int64_t)(taps - 1 + i) * C + c];
            keep[rr] = v;
        }
        for (int rr = 0; rr < taps - 1; ++rr) tl[(int64_t)rr * C + c] = keep[rr];
    }
}

static inline int dk_pad(int dk) { return dk <= 32 ? 32 : dk <= 64 ? 64 : dk <= 128 ? 128 : 256; }
static inline int dv_pad(int dv) { return dv <= 32 ? 32 : dv <= 64 ? 64 : dv <= 128 ? 128 : 256; }

template <typename T>
int launch_delta(const float* conv, int64_t C, const void* a, int64_t ld_a, const void* b, int64_t ld_b, const void* gate, int64_t ld_g,
                 const float* A_log, const float* dt_bias, const float* gain, float* state, float* tail, const void* proj, int64_t ld_p,
                 const int32_t* slots, const int32_t* cu_q, const int32_t* positions, void* out, int64_t ld_out, int B, int H, int G,
                 int dk, int dv, int taps, float eps, float unit_eps, float q_scale, hipStream_t st) {
    const int DKP = dk_pad(dk), DVP = dv_pad(dv), NT = DVP * RS;
    const int64_t head_floats = (int64_t)DKP * DVP;
    const size_t lds = ((size_t)3 * CH * (DKP + RS * 4) + (size_t)3 * CH * DVP + 2 * CH) * sizeof(float);
#define TGIS_DELTA_LAUNCH(DKT, DVT)                                                                                                       \
    do {                                                                                                                                  \
        if (lds > 48 * 1024)                                                                                                              \
            (void)hipFuncSetAttribute((const void*)delta_scan_kernel<T, DKT, DVT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
        hipLaunchKernelGGL((delta_scan_kernel<T, DKT, DVT>), dim3((unsigned)B, (unsigned)H), dim3(NT), lds, st, conv, C, (const T*)a, ld_a, \
                           (const T*)b, ld_b, (const T*)gate, ld_g, A_log, dt_bias, gain, state, head_floats, tail, (const T*)proj,        \
                           ld_p, slots, cu_q, positions, (T*)out, ld_out, H, G, dk, dv, taps, eps, unit_eps, q_scale);                     \
    } while (0)
#define TGIS_DELTA_DV(DKT)                            \
    do {                                              \
        if (DVP == 32) TGIS_DELTA_LAUNCH(DKT, 32);    \
        else if (DVP == 64) TGIS_DELTA_LAUNCH(DKT, 64);   \
        else if (DVP == 128) TGIS_DELTA_LAUNCH(DKT, 128); \
        else TGIS_DELTA_LAUNCH(DKT, 256);             \
    } while (0)
    if (DKP == 32)
        TGIS_DELTA_DV(32);
    else if (DKP == 64)
        TGIS_DELTA_DV(64);
    else if (DKP == 128)
        TGIS_DELTA_DV(128);
    else
        TGIS_DELTA_DV(256);
#undef TGIS_DELTA_DV
#undef TGIS_DELTA_LAUNCH
    return 0;
}

}  // namespace

static bool dtype3(int d) { return d == TGIS_F16 || d == TGIS_BF16 || d == TGIS_F32; }

// floats of one head's state in a slot (key rows and value columns padded to the scan kernel's tile)
extern "C" int64_t tgis_delta_state_floats(int dk, int dv) {
    if (dk < 1 || dk > 256 || dv < 1 || dv > 256) return -1;
    return (int64_t)dk_pad(dk) * dv_pad(dv);
}

extern "C" int tgis_short_conv_silu(const void* x, int64_t ld_x, const float* w, const float* tail, const int32_t* state_slots,
                                    const int32_t* cu_seqlens_q, const int32_t* positions, int64_t B, float* out, int64_t T,
                                    int64_t C, int taps, int dtype, void* stream) {
    TGIS_CHECK_ARG(x && w && tail && state_slots && cu_seqlens_q && positions && out, "tgis_short_conv_silu: null tensor");
    TGIS_CHECK_ARG(B >= 1 && C >= 1 && C <= 65535 * 256 && ld_x >= C && taps >= 1 && taps <= 9 && dtype3(dtype),
                   "tgis_short_conv_silu: bad arguments (taps 1 .. 9)");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    const int esz = dtype == TGIS_F32 ? 4 : 2;
    if (C % 4 == 0 && (ld_x * esz) % (4 * esz) == 0 && ((uintptr_t)x % (4 * esz)) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)tail % 16) == 0) {
        if (T >= 256 && taps >= 2 && taps <= 5) {
            dim3 rgrid((unsigned)cdiv64(T, TB), (unsigned)cdiv64(C / 4, 256));
#define TGIS_CONV_RUN(TT, TP) \
    hipLaunchKernelGGL((short_conv_silu_run_kernel<TT, TP>), rgrid, dim3(256), 0, st, (const TT*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, T, C)
#define TGIS_CONV_TAPS(TT)                     \
    do {                                       \
        if (taps == 2) TGIS_CONV_RUN(TT, 2);   \
        else if (taps == 3) TGIS_CONV_RUN(TT, 3); \
        else if (taps == 4) TGIS_CONV_RUN(TT, 4); \
        else TGIS_CONV_RUN(TT, 5);             \
    } while (0)
            if (dtype == TGIS_F16) TGIS_CONV_TAPS(f16);
            else if (dtype == TGIS_BF16) TGIS_CONV_TAPS(bf16);
            else TGIS_CONV_TAPS(float);
#undef TGIS_CONV_TAPS
#undef TGIS_CONV_RUN
            TGIS_CHECK_LAUNCH();
            return TGIS_OK;
        }
        dim3 vgrid((unsigned)T, (unsigned)cdiv64(C / 4, 256));
        if (dtype == TGIS_F16)
            hipLaunchKernelGGL(short_conv_silu_vec_kernel<f16>, vgrid, dim3(256), 0, st, (const f16*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, C, taps);
        else if (dtype == TGIS_BF16)
            hipLaunchKernelGGL(short_conv_silu_vec_kernel<bf16>, vgrid, dim3(256), 0, st, (const bf16*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, C, taps);
        else
            hipLaunchKernelGGL(short_conv_silu_vec_kernel<float>, vgrid, dim3(256), 0, st, (const float*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, C, taps);
        TGIS_CHECK_LAUNCH();
        return TGIS_OK;
    }
    dim3 grid((unsigned)T, (unsigned)cdiv64(C, 256));
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(short_conv_silu_kernel<f16>, grid, dim3(256), 0, st, (const f16*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, C, taps);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(short_conv_silu_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, C, taps);
    else
        hipLaunchKernelGGL(short_conv_silu_kernel<float>, grid, dim3(256), 0, st, (const float*)x, ld_x, w, tail, state_slots, cu_seqlens_q, positions, (int)B, out, C, taps);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// conv [T, C] fp32 = the convolved and activated q | k | v (G dk, G dk, H dv columns); a [T, H dk], b [T, H], gate [T, H dv] and
// proj [T, >= C] (the projection before the convolution, whose last rows become the slot's tail) in the activation dtype
extern "C" int tgis_delta_scan(const float* conv, int64_t C, const void* a, int64_t ld_a, const void* b, int64_t ld_b, const void* gate,
                               int64_t ld_gate, const float* A_log, const float* dt_bias, const float* gain, float* state, float* tail,
                               const void* proj, int64_t ld_proj, const int32_t* state_slots, const int32_t* cu_seqlens_q,
                               const int32_t* positions, void* out, int64_t ld_out, int64_t B, int H, int G, int dk, int dv, int taps,
                               float eps, float unit_eps, float q_scale, int dtype, void* stream) {
    TGIS_CHECK_ARG(conv && a && b && gate && A_log && dt_bias && gain && state && tail && proj && state_slots && cu_seqlens_q && positions && out,
                   "tgis_delta_scan: null tensor");
    TGIS_CHECK_ARG(B >= 1 && H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256,
                   "tgis_delta_scan: head geometry H %d, G %d, dk %d, dv %d (widths 1 .. 256, H a multiple of G)", H, G, dk, dv);
    TGIS_CHECK_ARG(C == (int64_t)2 * G * dk + (int64_t)H * dv && ld_a >= (int64_t)H * dk && ld_b >= H && ld_gate >= (int64_t)H * dv &&
                       ld_proj >= C && ld_out >= (int64_t)H * dv && taps >= 1 && taps <= 9 && dtype3(dtype),
                   "tgis_delta_scan: bad strides, taps (1 .. 9) or dtype");
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    if (dtype == TGIS_F16)
        launch_delta<f16>(conv, C, a, ld_a, b, ld_b, gate, ld_gate, A_log, dt_bias, gain, state, tail, proj, ld_proj, state_slots, cu_seqlens_q, positions, out, ld_out, (int)B, H, G, dk, dv, taps, eps, unit_eps, q_scale, st);
    else if (dtype == TGIS_BF16)
        launch_delta<bf16>(conv, C, a, ld_a, b, ld_b, gate, ld_gate, A_log, dt_bias, gain, state, tail, proj, ld_proj, state_slots, cu_seqlens_q, positions, out, ld_out, (int)B, H, G, dk, dv, taps, eps, unit_eps, q_scale, st);
    else
        launch_delta<float>(conv, C, a, ld_a, b, ld_b, gate, ld_gate, A_log, dt_bias, gain, state, tail, proj, ld_proj, state_slots, cu_seqlens_q, positions, out, ld_out, (int)B, H, G, dk, dv, taps, eps, unit_eps, q_scale, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
