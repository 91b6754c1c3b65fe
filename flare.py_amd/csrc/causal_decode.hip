// Recurrent decode of causal FLARE: N single-token steps in ONE launch, the state in registers throughout.
//
// Same definition, state and validation as causal_mfma.hip; a kernel of its own because a decode step has no
// matrix shape: per (b,h) and token it is M dot products of length D, M*D multiply-adds into the state and M*D
// for the output.  One workgroup of 8 waves per (b,h); wave w owns MW = M/8 latents and works in two lane maps:
//   score stage : lane = (latent ms = lane % MW, dp = lane / MW): a D/SL slice of <q_m, k_t> as packed dot
//                 products, summed over the SL = 64/MW lanes of a latent (measured faster than whole rows on
//                 MW lanes with the rest idle); then P = exp2(score - mu0), den += P,
//                 W = P * exp2(mu0 - cref) (one common shift for the softmax over latents), G = W / den;
//                 (P, G, W) of the wave's latents go through a wave-private LDS table (no barrier);
//   state stage : lane = (column d = lane % D, mp = lane / D): U[m,d] += P_m v_t[d] and sum_m G_m U[m,d] over the
//                 lane's ML = MW * D / 64 latents, plus sum_m W_m.
// The eight partial output rows and weight sums meet in LDS (double buffered: one barrier per step); the waves
// take turns to divide, validate (sum of weights inside 2^-60..2^120, finite output) and stores the row.  A (b,h) that
// fails validation has left its state untouched: its workgroup repeats the steps on the spot with a running maximum
// per latent (the exact path at the end of the kernel), so a call is one launch whatever the scores are.
#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLMin = 8.6736174e-19f, kLMax = 1.329228e36f;   // 2^-60, 2^120
constexpr int kDecWaves = 8;

template <typename T> struct Dt;
template <> struct Dt<bf16_t> {
    static __device__ __forceinline__ float dot2(uint32_t x, uint32_t y, float acc)
    {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, y), acc, false);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float unpack(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
    static __device__ __forceinline__ uint16_t bits(float v) { return f32_to_bf16_bits(v); }
};
template <> struct Dt<f16_t> {
    static __device__ __forceinline__ float dot2(uint32_t x, uint32_t y, float acc)
    {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, x), __builtin_bit_cast(f16x2, y), acc, false);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float unpack(uint16_t b) { return float(__builtin_bit_cast(_Float16, b)); }
    static __device__ __forceinline__ uint16_t bits(float v)
    {
        const _Float16 h = (_Float16)v;
        return __builtin_bit_cast(uint16_t, h);
    }
};

template <typename T, int D, int MW>
__global__ __launch_bounds__(64 * kDecWaves) void causal_decode_kernel(CausalArgs a)
{
    constexpr int NW = kDecWaves, M = NW * MW;
    constexpr int SL = 64 / MW;       // lanes per latent in the score stage
    constexpr int DS = D / SL;        // dims per lane there
    constexpr int QP = DS / 2;        // packed pairs per lane there
    constexpr int QV = QP / 4;        // 16-byte loads of k per lane and step
    constexpr int NP = 64 / D;        // lanes per column in the state stage
    constexpr int ML = MW / NP;       // latents per lane there
    static_assert(QP % 4 == 0 && ML >= 1 && (MW == 16 || MW == 32), "unsupported shape");
    using E = Dt<T>;

    __shared__ __attribute__((aligned(16))) float pgw[NW][MW][4];   // P, G, W of the wave's latents (one 16-byte read each)
    __shared__ float ypart[2][NW][D];
    __shared__ float rpart[4][NW];      // [2][NW] partial weight sums; the exact path keeps each step's largest score per wave behind them
    __shared__ int bad_flag;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
    const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H;
    const int N = a.N;
    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    uint16_t* y = (uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    float* mu_g = a.mu + (int64_t)bh * M;
    float* den_g = a.den + (int64_t)bh * M;
    float* num_g = a.num + (int64_t)bh * M * D;
    const float sl2 = a.scale * kLog2e;
    if (tid == 0) bad_flag = 0;

    // one shift for the softmax over latents: the largest per-latent shift of the incoming state
    float cref = kNegBig;
    for (int m = lane; m < M; m += 256) {          // up to four loads in flight (M <= 256: one round trip)
        float mu[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) mu[u] = mu_g[m + 64 * u < M ? m + 64 * u : m];
#pragma unroll
        for (int u = 0; u < 4; ++u) cref = fmaxf(cref, mu[u] <= kNegBig ? 0.f : mu[u] * kLog2e);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cref = fmaxf(cref, __shfl_xor(cref, o));

    // score stage: latent ms of the wave, dims dp * DS .. + DS
    const int ms = lane % MW, dp = lane / MW;
    const bool score_lane = dp == 0;
    const int m_s = w * MW + ms;
    uint32_t qp[QP];
    {
        const uint16_t* qr = q + (int64_t)m_s * a.qs[2] + dp * DS;
#pragma unroll
        for (int j = 0; j < QP; ++j) qp[j] = E::pack2(E::unpack(qr[2 * j]) * sl2, E::unpack(qr[2 * j + 1]) * sl2);
    }
    const float mu_in = mu_g[m_s];
    const bool fresh = mu_in <= kNegBig;
    const float mu0 = fresh ? 0.f : mu_in * kLog2e;
    const float fw = fast_exp2(mu0 - cref);
    const float den_in = den_g[m_s];       // read whether fresh or not: a load under the condition would wait for mu first
    float den = fresh ? 0.f : den_in;

    // state stage: column d, latents w * MW + mp * ML + j
    const int d = lane % D, mp = lane / D;
    float U[ML];
    {
        float mu_j[ML];
#pragma unroll
        for (int j = 0; j < ML; ++j) {
            const int m = w * MW + mp * ML + j;
            mu_j[j] = mu_g[m];
            U[j] = num_g[(int64_t)m * D + d];      // all loads in flight together; a fresh latent's sums are dropped below
        }
#pragma unroll
        for (int j = 0; j < ML; ++j) U[j] = mu_j[j] <= kNegBig ? 0.f : U[j];
    }

    // k_t and v_t arrive kPF steps ahead of their use: a step is shorter than the latency of the loads
    constexpr int kPF = 4;
    u32x4 kq[kPF][QV];
    uint16_t vq[kPF];
    auto fetch = [&](int n, u32x4 (&dst)[QV], uint16_t& vd) {
        const int nc = n < N ? n : N - 1;
        const uint16_t* kr = k + (int64_t)nc * a.ks[2] + dp * DS;
#pragma unroll
        for (int i = 0; i < QV; ++i) dst[i] = *reinterpret_cast<const u32x4*>(kr + 8 * i);
        vd = v[(int64_t)nc * a.vs[2] + d];
    };
#pragma unroll
    for (int u = 0; u < kPF; ++u) fetch(u, kq[u], vq[u]);

    bool bad = false;
    for (int n0 = 0; n0 < N; n0 += kPF) {
#pragma unroll
        for (int u = 0; u < kPF; ++u) {
            const int n = n0 + u;
            if (n >= N) break;
            const int buf = n & 1;

            // ---- score stage ----
            float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < QV; ++i)
#pragma unroll
                for (int c = 0; c < 4; ++c) s4[c] = E::dot2(qp[4 * i + c], kq[u][i][c], s4[c]);
            const float vd = E::unpack(vq[u]);
            fetch(n + kPF, kq[u], vq[u]);          // this slot is free again
            float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
            if constexpr (MW == 16) s = sum_xor16(s);
            s = sum_xor32(s);
            const float p = fast_exp2(s - mu0);
            den += p;
            const float wgt = p * fw;
            asm volatile("" ::: "memory");      // the lanes' stores and their reads of each other's entries keep their order
            if (score_lane) *reinterpret_cast<f32x4*>(&pgw[w][ms][0]) = f32x4{p, wgt * __builtin_amdgcn_rcpf(den), wgt, 0.f};
            asm volatile("" ::: "memory");

            // ---- state stage (the table is private to the wave: its reads follow its writes in program order) ----
            float acc4[4] = {0.f, 0.f, 0.f, 0.f}, rw4[4] = {0.f, 0.f, 0.f, 0.f};     // four short chains, not one long
#pragma unroll
            for (int j = 0; j < ML; ++j) {
                const f32x4 t = *reinterpret_cast<const f32x4*>(&pgw[w][mp * ML + j][0]);
                U[j] = fmaf(t[0], vd, U[j]);
                acc4[j & 3] = fmaf(t[1], U[j], acc4[j & 3]);
                rw4[j & 3] += t[2];
            }
            float acc = (acc4[0] + acc4[1]) + (acc4[2] + acc4[3]), rw = (rw4[0] + rw4[1]) + (rw4[2] + rw4[3]);
            if constexpr (NP == 2) {
                acc = sum_xor32(acc);
                rw = sum_xor32(rw);
            }
            if (mp == 0) ypart[buf][w][d] = acc;
            if (lane == 0) rpart[buf][w] = rw;
            __syncthreads();

            // ---- one wave (they take turns): sum over the waves, divide, validate, store ----
            if (w == (n & (NW - 1)) && lane < D) {
                float ys = 0.f, r = 0.f;
#pragma unroll
                for (int i = 0; i < NW; ++i) {
                    ys += ypart[buf][i][lane];
                    r += rpart[buf][i];
                }
                const float o = ys * __builtin_amdgcn_rcpf(r);
                bad = bad || !(r >= kLMin && r <= kLMax) || !(fabsf(o) <= 3.0e38f);
                y[(int64_t)n * a.ys[2] + lane] = E::bits(o);
                if (a.lse && lane == 0) a.lse[(int64_t)bh * N + n] = (cref + __log2f(r)) * kLn2;
            }
        }
    }

    bad = bad || !(den >= kLMin && den <= kLMax);
    if (__any(bad) && lane == 0) bad_flag = 1;
    __syncthreads();
    if (bad_flag) {
        // Exact path, in the same launch: the workgroup repeats all N steps from the incoming state (nothing of it has
        // been overwritten) with a running maximum per latent, scores in fp32 from the unrounded latents, and the
        // softmax over the latents shifted by each step's own largest score.  Same two lane maps; the step's largest
        // score crosses the waves through LDS, which costs a second barrier per step.
        float* cmax = &rpart[0][0] + 2 * NW;      // [2][NW], behind rpart (declared below as one array of 4 NW floats)
        float qf[DS];
        {
            const uint16_t* qr = q + (int64_t)m_s * a.qs[2] + dp * DS;
#pragma unroll
            for (int j = 0; j < DS; ++j) qf[j] = E::unpack(qr[j]);
        }
        float mu2 = fresh ? kNegBig : mu_in * kLog2e;
        den = fresh ? 0.f : den_in;
        {
            float mu_j[ML];
#pragma unroll
            for (int j = 0; j < ML; ++j) {
                const int m = w * MW + mp * ML + j;
                mu_j[j] = mu_g[m];
                U[j] = num_g[(int64_t)m * D + d];
            }
#pragma unroll
            for (int j = 0; j < ML; ++j) U[j] = mu_j[j] <= kNegBig ? 0.f : U[j];
        }
        for (int n = 0; n < N; ++n) {
            const int buf = n & 1;
            const uint16_t* kr = k + (int64_t)n * a.ks[2] + dp * DS;
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < DS; ++j) s = fmaf(qf[j], E::unpack(kr[j]), s);
            if constexpr (MW == 16) s = sum_xor16(s);
            s = sum_xor32(s) * sl2;
            const float mun = fmaxf(mu2, s);
            const float al = fast_exp2(mu2 - mun), p = fast_exp2(s - mun);
            den = fmaf(al, den, p);
            mu2 = mun;
            float cm = s;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) cm = fmaxf(cm, __shfl_xor(cm, o));
            if (lane == 0) cmax[buf * NW + w] = cm;
            asm volatile("" ::: "memory");
            if (score_lane) *reinterpret_cast<f32x4*>(&pgw[w][ms][0]) = f32x4{al, p, s, 1.f / den};
            asm volatile("" ::: "memory");
            __syncthreads();
            float c = cmax[buf * NW];
#pragma unroll
            for (int i = 1; i < NW; ++i) c = fmaxf(c, cmax[buf * NW + i]);
            const float vd = E::unpack(v[(int64_t)n * a.vs[2] + d]);
            float acc = 0.f, rw = 0.f;
#pragma unroll
            for (int j = 0; j < ML; ++j) {
                const f32x4 t = *reinterpret_cast<const f32x4*>(&pgw[w][mp * ML + j][0]);
                U[j] = fmaf(t[1], vd, t[0] * U[j]);
                const float wgt = fast_exp2(t[2] - c);
                acc = fmaf(wgt * t[3], U[j], acc);
                rw += wgt;
            }
            if constexpr (NP == 2) {
                acc = sum_xor32(acc);
                rw = sum_xor32(rw);
            }
            if (mp == 0) ypart[buf][w][d] = acc;
            if (lane == 0) rpart[buf][w] = rw;
            __syncthreads();
            if (w == (n & (NW - 1)) && lane < D) {
                float ys = 0.f, r = 0.f;
#pragma unroll
                for (int i = 0; i < NW; ++i) {
                    ys += ypart[buf][i][lane];
                    r += rpart[buf][i];
                }
                y[(int64_t)n * a.ys[2] + lane] = E::bits(ys / r);
                if (a.lse && lane == 0) a.lse[(int64_t)bh * N + n] = (c + __log2f(r)) * kLn2;
            }
        }
        if (score_lane) {
            mu_g[m_s] = mu2 * kLn2;
            den_g[m_s] = den;
        }
#pragma unroll
        for (int j = 0; j < ML; ++j) num_g[(int64_t)(w * MW + mp * ML + j) * D + d] = U[j];
        return;
    }
    if (score_lane) {
        mu_g[m_s] = mu0 * kLn2;
        den_g[m_s] = den;
    }
#pragma unroll
    for (int j = 0; j < ML; ++j) num_g[(int64_t)(w * MW + mp * ML + j) * D + d] = U[j];
}

template <typename T>
hipError_t launch_t(const CausalArgs& a, hipStream_t st)
{
    dim3 grid(a.B * a.H), block(64 * kDecWaves);
    if (a.M == 128 && a.D == 64)      hipLaunchKernelGGL((causal_decode_kernel<T, 64, 16>), grid, block, 0, st, a);
    else if (a.M == 128 && a.D == 32) hipLaunchKernelGGL((causal_decode_kernel<T, 32, 16>), grid, block, 0, st, a);
    else if (a.M == 256 && a.D == 32) hipLaunchKernelGGL((causal_decode_kernel<T, 32, 32>), grid, block, 0, st, a);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace

hipError_t launch_causal_decode_steps(const CausalArgs& a, int dtype, hipStream_t st)
{
    return dtype == 1 ? launch_t<bf16_t>(a, st) : launch_t<f16_t>(a, st);
}

}  // namespace flare
