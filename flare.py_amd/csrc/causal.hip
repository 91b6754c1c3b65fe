// Causal FLARE: chunked prefill and recurrent decode, fp32 arithmetic, state resident in LDS.
//
// Definition (the reference names causal FLARE in README.md:60 but holds no code for it;
// the chunk structure follows lra/models/triton/causal_linear.py:81-137 with the plain sum
// replaced by the online-softmax triple):
//   sigma[t,m] = s <q_m, k_t>
//   z_t[m]     = sum_{tau<=t} softmax over tau<=t of sigma[.,m] applied to v
//   y_t        = sum_m softmax_m(sigma[t,.])_m z_t[m]
// State per (b,h): mu[M] (max), den[M], num[M,D], with z_t = num/den.
//
// One workgroup owns one (b,h) and walks its tokens in blocks of TB tokens; the state never
// leaves LDS between blocks, so N decode steps (TB = 1) cost one launch.
// Inside a block every token keeps its own per-latent running maximum (the intra-block weights
// are exp2(sigma[tau,m] - mc_t[m]) with tau <= t, so no exponent is ever positive), which makes the
// kernel exact for arbitrary score jumps at the price of TB*TB*M/2 extra exponentials per block.
#include "common.hpp"

namespace flare {

namespace {

constexpr int kThreads = 256;

struct CausalLds {
    int q, U, sg, gg, mct, cf, ks, vs, As, mu, den, al, rmax, rinv, total;  // offsets in floats
};

__host__ __device__ inline CausalLds causal_lds_layout(int M, int D, int TB)
{
    CausalLds L;
    int o = 0;
    L.q = o;    o += M * (D + 1);
    L.U = o;    o += M * D;
    L.sg = o;   o += TB * (M + 1);
    L.gg = o;   o += TB * (M + 1);
    L.mct = o;  o += TB * (M + 1);
    L.cf = o;   o += TB * (M + 1);
    L.ks = o;   o += TB * D;
    L.vs = o;   o += TB * D;
    L.As = o;   o += TB * TB;
    L.mu = o;   o += M;
    L.den = o;  o += M;
    L.al = o;   o += M;
    L.rmax = o; o += TB;
    L.rinv = o; o += TB;
    L.total = o;
    return L;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

template <typename T, int TB>
__global__ __launch_bounds__(kThreads) void causal_generic_kernel(CausalArgs a)
{
    extern __shared__ float sm[];
    const int M = a.M, D = a.D, N = a.N;
    const CausalLds L = causal_lds_layout(M, D, TB);
    float* qs = sm + L.q;   float* U = sm + L.U;   float* sg = sm + L.sg; float* gg = sm + L.gg;
    float* mct = sm + L.mct; float* cf = sm + L.cf;
    float* ks = sm + L.ks;  float* vs = sm + L.vs; float* As = sm + L.As;
    float* mu_s = sm + L.mu; float* den_s = sm + L.den; float* al_s = sm + L.al;
    float* rmax = sm + L.rmax; float* rinv = sm + L.rinv;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H;
    if (a.flags != nullptr && a.flags[bh] == 0) {
        // Launched behind the matrix-core kernels: only marked (b,h) are redone.  For the others a prefill in several
        // segments has staged its final state in the last workspace slot; it becomes (mu, den, num) here,
        // once every segment is known to have passed (a fresh state's shift becomes 0).
        if (a.n_segs > 1) {
            const int M = a.M, D = a.D;
            const float* sd = a.seg_den + ((int64_t)bh * a.n_slots + a.n_slots - 1) * M;
            const float* sn = a.seg_num + ((int64_t)bh * a.n_slots + a.n_slots - 1) * M * D;
            float* num = a.num + (int64_t)bh * M * D;
            for (int i = tid; i < M; i += kThreads) {
                const float mu = a.mu[(int64_t)bh * M + i];
                a.mu[(int64_t)bh * M + i] = mu <= kNegBig ? 0.f : mu;
                a.den[(int64_t)bh * M + i] = sd[i];
            }
            if (((reinterpret_cast<uintptr_t>(num) | reinterpret_cast<uintptr_t>(sn)) & 15) == 0 && (M * D) % 4 == 0) {
                for (int i = tid; i < M * D / 4; i += kThreads)
                    reinterpret_cast<float4*>(num)[i] = reinterpret_cast<const float4*>(sn)[i];
            } else {
                for (int i = tid; i < M * D; i += kThreads) num[i] = sn[i];
            }
        }
        return;
    }
    const T* q = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
    const T* k = (const T*)a.k + b * a.ks[0] + h * a.ks[1];
    const T* v = (const T*)a.v + b * a.vs[0] + h * a.vs[1];
    T* y = (T*)a.y + b * a.ys[0] + h * a.ys[1];
    float* mu_g = a.mu + (int64_t)bh * M;
    float* den_g = a.den + (int64_t)bh * M;
    float* num_g = a.num + (int64_t)bh * M * D;
    const float sl2 = a.scale * kLog2e;

    for (int idx = tid; idx < M * D; idx += kThreads) {
        const int m = idx / D, d = idx - m * D;
        qs[m * (D + 1) + d] = to_f32(q[(int64_t)m * a.qs[2] + d]) * sl2;
        const float mu = mu_g[m], un = num_g[idx];
        U[idx] = mu <= kNegBig ? 0.f : un;                   // a fresh latent's sums are dropped (they may be uninitialised)
    }
    for (int m = tid; m < M; m += kThreads) {
        const float mu = mu_g[m], dn = den_g[m];
        mu_s[m] = mu <= kNegBig ? kNegBig : mu * kLog2e;
        den_s[m] = mu <= kNegBig ? 0.f : dn;
    }

    for (int n0 = 0; n0 < N; n0 += TB) {
        const int tb = min(TB, N - n0);
        __syncthreads();
        for (int idx = tid; idx < tb * D; idx += kThreads) {
            const int t = idx / D, d = idx - t * D;
            ks[idx] = to_f32(k[(int64_t)(n0 + t) * a.ks[2] + d]);
            vs[idx] = to_f32(v[(int64_t)(n0 + t) * a.vs[2] + d]);
        }
        __syncthreads();
        // scores (log2 units)
        for (int idx = tid; idx < tb * M; idx += kThreads) {
            const int t = idx / M, m = idx - t * M;
            float s = 0.f;
            for (int d = 0; d < D; ++d) s = fmaf(ks[t * D + d], qs[m * (D + 1) + d], s);
            sg[t * (M + 1) + m] = s;
        }
        __syncthreads();
        // softmax statistics over the latents of each token
        for (int t = wave; t < tb; t += kThreads / 64) {
            float mx = kNegBig;
            for (int m = lane; m < M; m += 64) mx = fmaxf(mx, sg[t * (M + 1) + m]);
            mx = wave_max(mx);
            float sum = 0.f;
            for (int m = lane; m < M; m += 64) sum += fast_exp2(sg[t * (M + 1) + m] - mx);
            sum = wave_sum(sum);
            if (lane == 0) {
                rmax[t] = mx;
                rinv[t] = 1.f / sum;
                if (a.lse) a.lse[(int64_t)bh * N + n0 + t] = (mx + __log2f(sum)) * kLn2;
            }
        }
        __syncthreads();
        // per latent, token by token: running maximum mc_t, denominator relative to it,
        // G = w / den_t and the coefficient of the carried-in state exp2(mu - mc_t) G
        for (int m = tid; m < M; m += kThreads) {
            const float mp = mu_s[m];
            float mc = mp, dc = den_s[m];
            for (int t = 0; t < tb; ++t) {
                const float s = sg[t * (M + 1) + m];
                const float mn = fmaxf(mc, s);
                dc = dc * fast_exp2(mc - mn) + fast_exp2(s - mn);
                mc = mn;
                const float w = fast_exp2(s - rmax[t]) * rinv[t];
                const float gv = w / dc;
                gg[t * (M + 1) + m] = gv;
                mct[t * (M + 1) + m] = mc;
                cf[t * (M + 1) + m] = gv * fast_exp2(mp - mc);
            }
            mu_s[m] = mc; den_s[m] = dc; al_s[m] = fast_exp2(mp - mc);
        }
        __syncthreads();
        // A[t][tau] = sum_m G[t,m] exp2(sigma[tau,m] - mc_t[m]) for tau <= t (every exponent <= 0)
        if (TB > 1) {
            for (int idx = tid; idx < tb * tb; idx += kThreads) {
                const int t = idx / tb, tau = idx - t * tb;
                float acc = 0.f;
                if (tau <= t)
                    for (int m = 0; m < M; ++m)
                        acc = fmaf(gg[t * (M + 1) + m], fast_exp2(sg[tau * (M + 1) + m] - mct[t * (M + 1) + m]), acc);
                As[t * TB + tau] = acc;
            }
            __syncthreads();
        }
        // y[t,d] = sum_m cf[t,m] U[m,d] + sum_{tau<=t} A[t,tau] v[tau,d]
        for (int idx = tid; idx < tb * D; idx += kThreads) {
            const int t = idx / D, d = idx - t * D;
            float acc = 0.f;
            for (int m = 0; m < M; ++m) acc = fmaf(cf[t * (M + 1) + m], U[m * D + d], acc);
            if (TB > 1) {
                for (int tau = 0; tau <= t; ++tau) acc = fmaf(As[t * TB + tau], vs[tau * D + d], acc);
            } else {
                // single token: A[0][0] = sum_m G[0,m] exp2(sigma[0,m] - mc_0[m])
                float a00 = 0.f;
                for (int m = 0; m < M; ++m) a00 = fmaf(gg[m], fast_exp2(sg[m] - mct[m]), a00);
                acc = fmaf(a00, vs[d], acc);
            }
            y[(int64_t)(n0 + t) * a.ys[2] + d] = from_f32<T>(acc);
        }
        __syncthreads();
        // probabilities relative to the end-of-block maximum, in place of the scores
        for (int idx = tid; idx < tb * M; idx += kThreads) {
            const int t = idx / M, m = idx - t * M;
            sg[t * (M + 1) + m] = fast_exp2(sg[t * (M + 1) + m] - mu_s[m]);
        }
        __syncthreads();
        // U[m,d] = alpha[m] U[m,d] + sum_t P[t,m] v[t,d]
        for (int idx = tid; idx < M * D; idx += kThreads) {
            const int m = idx / D, d = idx - m * D;
            float u = al_s[m] * U[idx];
            for (int t = 0; t < tb; ++t) u = fmaf(sg[t * (M + 1) + m], vs[t * D + d], u);
            U[idx] = u;
        }
    }
    __syncthreads();
    for (int idx = tid; idx < M * D; idx += kThreads) num_g[idx] = U[idx];
    for (int m = tid; m < M; m += kThreads) {
        mu_g[m] = mu_s[m] <= kNegBig ? -INFINITY : mu_s[m] * kLn2;
        den_g[m] = den_s[m];
    }
}

template <typename T, int TB>
hipError_t launch_tb(const CausalArgs& a, hipStream_t st)
{
    const CausalLds L = causal_lds_layout(a.M, a.D, TB);
    const size_t lds = (size_t)L.total * sizeof(float);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    auto kern = causal_generic_kernel<T, TB>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(a.B * a.H), dim3(kThreads), lds, st, a);
    return hipGetLastError();
}

template <int TB>
hipError_t launch_dt(const CausalArgs& a, int dtype, hipStream_t st)
{
    switch (dtype) {
        case 0: return launch_tb<float, TB>(a, st);
        case 1: return launch_tb<bf16_t, TB>(a, st);
        default: return launch_tb<f16_t, TB>(a, st);
    }
}

// Joins latent groups that ran as causal problems of their own: y[r,:] = sum_g w_g y_g[r,:] with
// w_g = exp(lse_g[r]) / sum_g' exp(lse_g'[r]).  One thread per 8 consecutive elements of a row, moved as 16-byte
// pieces (one for a 16-bit type, two for fp32); fp32 arithmetic, groups visited in order (bit-stable).
template <typename T> __device__ __forceinline__ void join_load8(const T* p, float (&x)[8])
{
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    if constexpr (sizeof(T) == 4) {
        const u4 lo = *reinterpret_cast<const u4*>(p), hi = *reinterpret_cast<const u4*>(p + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[e] = __uint_as_float(lo[e]);
            x[4 + e] = __uint_as_float(hi[e]);
        }
    } else {
        const u4 raw = *reinterpret_cast<const u4*>(p);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint16_t b0 = uint16_t(raw[e] & 0xffffu), b1 = uint16_t(raw[e] >> 16);
            x[2 * e] = to_f32(__builtin_bit_cast(T, b0));
            x[2 * e + 1] = to_f32(__builtin_bit_cast(T, b1));
        }
    }
}
template <typename T> __device__ __forceinline__ void join_store8(T* p, const float (&x)[8])
{
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<u4*>(p) = u4{__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
        *reinterpret_cast<u4*>(p + 4) = u4{__float_as_uint(x[4]), __float_as_uint(x[5]), __float_as_uint(x[6]), __float_as_uint(x[7])};
    } else {
        u4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const T lo = from_f32<T>(x[2 * e]), hi = from_f32<T>(x[2 * e + 1]);
            o[e] = uint32_t(__builtin_bit_cast(uint16_t, lo)) | (uint32_t(__builtin_bit_cast(uint16_t, hi)) << 16);
        }
        *reinterpret_cast<u4*>(p) = o;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void causal_join_kernel(CausalJoinArgs a)
{
    const int per_row = a.D / 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= a.rows * per_row) return;
    const int64_t r = idx / per_row;
    const int c = (int)(idx - r * per_row) * 8;
    float mx = -INFINITY;
    for (int g = 0; g < a.n_groups; ++g) mx = fmaxf(mx, a.lse[g][r]);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float sum = 0.f;
    for (int g = 0; g < a.n_groups; ++g) {
        const float w = __expf(a.lse[g][r] - mx);
        sum += w;
        float x[8];
        join_load8((const T*)a.yg[g] + r * a.D + c, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(w, x[e], acc[e]);
    }
    const float inv = 1.f / sum;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= inv;
    join_store8((T*)a.y + r * a.D + c, acc);
}

}  // namespace

hipError_t launch_causal_join(const CausalJoinArgs& a, int dtype, hipStream_t st)
{
    const int64_t threads = a.rows * (a.D / 8);
    dim3 grid((unsigned)((threads + 255) / 256));
    switch (dtype) {
        case 0: hipLaunchKernelGGL(causal_join_kernel<float>, grid, dim3(256), 0, st, a); break;
        case 1: hipLaunchKernelGGL(causal_join_kernel<bf16_t>, grid, dim3(256), 0, st, a); break;
        default: hipLaunchKernelGGL(causal_join_kernel<f16_t>, grid, dim3(256), 0, st, a); break;
    }
    return hipGetLastError();
}

size_t causal_lds_bytes(int M, int D, bool decode)
{
    return (size_t)causal_lds_layout(M, D, decode ? 1 : 16).total * sizeof(float);
}

hipError_t launch_causal_prefill(const CausalArgs& a, int dtype, hipStream_t st) { return launch_dt<16>(a, dtype, st); }
hipError_t launch_causal_decode(const CausalArgs& a, int dtype, hipStream_t st) { return launch_dt<1>(a, dtype, st); }

}  // namespace flare
