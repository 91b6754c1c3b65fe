// Causal linear attention  y_t = (1/N) sum_{tau <= t} <q_t, k_tau> v_tau   (fp32 arithmetic).
//
// Definition: the token recurrence of lra/models/triton/causal_linear.py:317-336 (S += v k^T with
// k and v each scaled by N^-1/2, y_t = S q_t).  Structure: the three phases of
// causal_linear.py:81-137 / 338-389 — local states of token segments, an exclusive prefix over
// the segments, then per segment the inter-segment term q_t S plus the masked intra-tile term
// tril(Q K^T) V — with plain fixed-order sums (no atomics), so results are bit-stable.
//
// A segment is a run of 64-token tiles handled by one workgroup.  Inside a tile every thread
// owns one output column j and a fixed set of rows, for both the output (rows = tokens) and the
// state update (rows = key features), so the running state of a segment is read-modify-written
// in place in the workspace by the thread that owns each element.
#include "common.hpp"

namespace flare {

namespace {

constexpr int kTile = 64;   // tokens per tile

template <typename T>
__device__ __forceinline__ void load_rows(float* dst, int dst_stride, const T* src, int64_t row_stride,
                                          int n0, int n_end, int width, int tid)
{
    // rows n0 .. n0+63 of a [*, width] matrix into LDS as fp32; rows beyond n_end become 0
    for (int idx = tid; idx < kTile * width; idx += 256) {
        const int r = idx / width, c = idx % width;
        const int n = n0 + r;
        dst[r * dst_stride + c] = n < n_end ? to_f32(src[(int64_t)n * row_stride + c]) : 0.f;
    }
}

// DVP = Dv rounded up to a power of two in 4..128.  Thread tid owns column j = tid % DVP and the
// rows tg, tg + G, tg + 2G, ... with tg = tid / DVP, G = 256 / DVP.
template <typename T, int DVP, bool STATE_ONLY>
__global__ __launch_bounds__(256) void causal_linear_kernel(CausalLinearArgs a)
{
    constexpr int G = 256 / DVP;
    constexpr int RT = kTile / G;          // token rows per thread
    constexpr int RS = (128 + G - 1) / G;  // key-feature rows per thread (Dk <= 128)
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int Dk = a.Dk, Dv = a.Dv, KS = Dk + 1;
    float* qc = sm;                       // [64][Dk]
    float* kc = qc + kTile * Dk;          // [64][Dk+1]  (odd stride: conflict-free column walks)
    float* vc = kc + kTile * KS;          // [64][Dv]
    float* am = vc + kTile * Dv;          // [64][65]    tril(Q K^T)

    const int tid = threadIdx.x, j = tid % DVP, tg = tid / DVP;
    const int seg = blockIdx.x, bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const T* q = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
    const T* k = (const T*)a.k + b * a.ks[0] + h * a.ks[1];
    const T* v = (const T*)a.v + b * a.vs[0] + h * a.vs[1];
    T* y = (T*)a.y + b * a.ys[0] + h * a.ys[1];
    float* S = a.states + ((int64_t)bh * a.n_segs + seg) * Dk * Dv;   // this segment's slot
    const int n_lo = seg * a.seg_len, n_hi = min(a.N, n_lo + a.seg_len);
    const bool col = j < Dv;

    float sacc[RS];
#pragma unroll
    for (int r = 0; r < RS; ++r) sacc[r] = 0.f;

    for (int n0 = n_lo; n0 < n_hi; n0 += kTile) {
        __syncthreads();   // the previous tile's LDS reads are done
        load_rows(kc, KS, k, a.ks[2], n0, n_hi, Dk, tid);
        load_rows(vc, Dv, v, a.vs[2], n0, n_hi, Dv, tid);
        if (!STATE_ONLY) load_rows(qc, Dk, q, a.qs[2], n0, n_hi, Dk, tid);
        __syncthreads();

        if constexpr (!STATE_ONLY) {
            // am[t][tau] = <q_t, k_tau> for tau <= t, else 0
            for (int idx = tid; idx < kTile * kTile; idx += 256) {
                const int t = idx / kTile, tau = idx % kTile;
                float s = 0.f;
                if (tau <= t)
                    for (int i = 0; i < Dk; ++i) s = fmaf(qc[t * Dk + i], kc[tau * KS + i], s);
                am[t * (kTile + 1) + tau] = s;
            }
            __syncthreads();
            if (col) {
                float acc[RT];
#pragma unroll
                for (int r = 0; r < RT; ++r) acc[r] = 0.f;
                // inter-segment and earlier tiles: q_t S  (S is the running state in the workspace)
                for (int i = 0; i < Dk; ++i) {
                    const float s = S[(int64_t)i * Dv + j];
#pragma unroll
                    for (int r = 0; r < RT; ++r) acc[r] = fmaf(qc[(tg + r * G) * Dk + i], s, acc[r]);
                }
                // this tile: tril(Q K^T) V
                for (int tau = 0; tau < kTile; ++tau) {
                    const float vv = vc[tau * Dv + j];
#pragma unroll
                    for (int r = 0; r < RT; ++r) acc[r] = fmaf(am[(tg + r * G) * (kTile + 1) + tau], vv, acc[r]);
                }
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    const int n = n0 + tg + r * G;
                    if (n < n_hi) y[(int64_t)n * a.ys[2] + j] = from_f32<T>(acc[r] * a.inv_n);
                }
            }
            __syncthreads();   // every read of S for this tile is done before it is advanced
        }

        // state update S[i][j] += sum_tau k[tau][i] v[tau][j] for the rows this thread owns
        if (col) {
            float upd[RS];
#pragma unroll
            for (int r = 0; r < RS; ++r) upd[r] = 0.f;
            for (int tau = 0; tau < kTile; ++tau) {
                const float vv = vc[tau * Dv + j];
#pragma unroll
                for (int r = 0; r < RS; ++r) {
                    const int i = tg + r * G;
                    if (i < Dk) upd[r] = fmaf(kc[tau * KS + i], vv, upd[r]);
                }
            }
            if constexpr (STATE_ONLY) {
#pragma unroll
                for (int r = 0; r < RS; ++r) sacc[r] += upd[r];
            } else if (n0 + kTile < n_hi) {
#pragma unroll
                for (int r = 0; r < RS; ++r) {
                    const int i = tg + r * G;
                    if (i < Dk) S[(int64_t)i * Dv + j] += upd[r];
                }
            }
        }
    }
    if constexpr (STATE_ONLY) {
        if (col) {
#pragma unroll
            for (int r = 0; r < RS; ++r) {
                const int i = tg + r * G;
                if (i < Dk) S[(int64_t)i * Dv + j] = sacc[r];
            }
        }
    }
}

// Exclusive prefix over the segment slots of one (b,h): slot s := sum of the local states of
// segments < s.  The last segment's local state is never needed and its slot is only written.
__global__ __launch_bounds__(256) void causal_linear_prefix_kernel(CausalLinearArgs a)
{
    const int e = blockIdx.x * 256 + threadIdx.x, bh = blockIdx.y;
    const int sz = a.Dk * a.Dv;
    if (e >= sz) return;
    float* S = a.states + (int64_t)bh * a.n_segs * sz + e;
    // eight slots read before the first of them is overwritten: one trip to memory per eight segments
    float run = 0.f;
    for (int s0 = 0; s0 < a.n_segs; s0 += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = S[(int64_t)min(s0 + u, a.n_segs - 1) * sz];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int s = s0 + u;
            if (s < a.n_segs) {
                S[(int64_t)s * sz] = run;
                run += s + 1 < a.n_segs ? t[u] : 0.f;
            }
        }
    }
}

size_t lds_bytes(int Dk, int Dv) { return sizeof(float) * (size_t)kTile * (Dk + (Dk + 1) + Dv + (kTile + 1)); }

template <typename T, int DVP>
hipError_t launch_dvp(const CausalLinearArgs& a, hipStream_t st)
{
    const size_t lds = lds_bytes(a.Dk, a.Dv);
    const int BH = a.B * a.H;
    auto state_k = causal_linear_kernel<T, DVP, true>;
    auto out_k = causal_linear_kernel<T, DVP, false>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(state_k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(out_k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    if (a.n_segs > 1) hipLaunchKernelGGL(state_k, dim3(a.n_segs - 1, BH), dim3(256), lds, st, a);
    hipLaunchKernelGGL(causal_linear_prefix_kernel, dim3((a.Dk * a.Dv + 255) / 256, BH), dim3(256), 0, st, a);
    hipLaunchKernelGGL(out_k, dim3(a.n_segs, BH), dim3(256), lds, st, a);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_t(const CausalLinearArgs& a, hipStream_t st)
{
    if (a.Dv <= 4)   return launch_dvp<T, 4>(a, st);
    if (a.Dv <= 8)   return launch_dvp<T, 8>(a, st);
    if (a.Dv <= 16)  return launch_dvp<T, 16>(a, st);
    if (a.Dv <= 32)  return launch_dvp<T, 32>(a, st);
    if (a.Dv <= 64)  return launch_dvp<T, 64>(a, st);
    if (a.Dv <= 128) return launch_dvp<T, 128>(a, st);
    return hipErrorInvalidValue;
}

}  // namespace

int causal_linear_tile() { return kTile; }

hipError_t launch_causal_linear_prefix(const CausalLinearArgs& a, hipStream_t st)
{
    hipLaunchKernelGGL(causal_linear_prefix_kernel, dim3((a.Dk * a.Dv + 255) / 256, a.B * a.H), dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_causal_linear(const CausalLinearArgs& a, int dtype, hipStream_t st)
{
    if (a.Dk > 128 || a.Dv > 128) return hipErrorInvalidValue;
    if (dtype == 0) return launch_t<float>(a, st);
    if (dtype == 1) return launch_t<bf16_t>(a, st);
    return launch_t<f16_t>(a, st);
}

}  // namespace flare
