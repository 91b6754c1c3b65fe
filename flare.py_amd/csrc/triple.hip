// Triple (third-order) linear attention, fp32 FMA kernels.
//
//   state[i,j,k] = (1/N) sum_n f(k1)[n,i] v[n,j] f(k2)[n,k]
//   out[n,j]     = sum_{i,k} f(q1)[n,i] state[i,j,k] f(q2)[n,k]
// following TripleAttention.attn_einsum (lra/models/backends.py:1285-1292 of the reference) and
// TripleAttentionFunction.forward (lra/models/triton/triple.py:29-121), f = identity or elu+1
// (lra/models/kernels.py:23-24).  Where the reference accumulates the state with float
// atomics (triple.py:378), this build writes split-N partials and merges them in a fixed
// order, so results are bit-stable from run to run.
// With normalize the output is divided by the same contraction with v == 1, for which the
// state kernel also accumulates kk[i,k] = (1/N) sum_n f(k1)[n,i] f(k2)[n,k].
#include "common.hpp"

namespace flare {

namespace {

constexpr int kThreads = 256;
constexpr int kTile = 32;

__device__ __forceinline__ float feat(float x, int fm)
{
    if (!fm) return x;
    return x > 0.f ? x + 1.f : __expf(x);
}

// grid.x = n_splits * iblocks.  A workgroup owns IB rows i of the state (IB * Dv <= 256
// (i,j) pairs, one per thread) and every k; DQ bounds Dq at compile time.
template <typename T, int DQ>
__global__ __launch_bounds__(kThreads) void triple_state_kernel(TripleArgs a, int IB)
{
    __shared__ float k1s[kTile][DQ];
    __shared__ float k2s[kTile][DQ];
    __shared__ float vs[kTile][64];

    const int tid = threadIdx.x;
    const int Dq = a.Dq, Dv = a.Dv;
    const int iblocks = (Dq + IB - 1) / IB;
    const int split = blockIdx.x / iblocks, ib = blockIdx.x % iblocks;
    const int h = blockIdx.y, b = blockIdx.z;
    const int il = tid / Dv, j = tid - il * Dv;
    const int i = ib * IB + il;
    const bool live = il < IB && i < Dq;

    const T* k1 = (const T*)a.k1 + b * a.k1s[0] + h * a.k1s[1];
    const T* k2 = (const T*)a.k2 + b * a.k2s[0] + h * a.k2s[1];
    const T* v = (const T*)a.v + b * a.vs[0] + h * a.vs[1];

    float acc[DQ], kk[DQ];
#pragma unroll
    for (int k = 0; k < DQ; ++k) { acc[k] = 0.f; kk[k] = 0.f; }

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    for (int n0 = n_begin; n0 < n_end; n0 += kTile) {
        const int tn = min(kTile, n_end - n0);
        __syncthreads();
        for (int idx = tid; idx < tn * Dq; idx += kThreads) {
            const int t = idx / Dq, d = idx - t * Dq;
            k1s[t][d] = feat(to_f32(k1[(int64_t)(n0 + t) * a.k1s[2] + d]), a.feature_map);
            k2s[t][d] = feat(to_f32(k2[(int64_t)(n0 + t) * a.k2s[2] + d]), a.feature_map);
        }
        for (int idx = tid; idx < tn * Dv; idx += kThreads) {
            const int t = idx / Dv, d = idx - t * Dv;
            vs[t][d] = to_f32(v[(int64_t)(n0 + t) * a.vs[2] + d]);
        }
        __syncthreads();
        if (live) {
            for (int t = 0; t < tn; ++t) {
                const float ki = k1s[t][i];
                const float av = ki * vs[t][j];
#pragma unroll
                for (int k = 0; k < DQ; ++k)
                    if (k < Dq) acc[k] = fmaf(av, k2s[t][k], acc[k]);
                if (a.normalize && j == 0) {
#pragma unroll
                    for (int k = 0; k < DQ; ++k)
                        if (k < Dq) kk[k] = fmaf(ki, k2s[t][k], kk[k]);
                }
            }
        }
    }
    if (live) {
        const size_t per = (size_t)Dq * Dv * Dq + (size_t)Dq * Dq;
        float* part = a.part + (((size_t)b * a.H + h) * a.n_parts + split) * per;
        for (int k = 0; k < Dq; ++k) part[((size_t)i * Dv + j) * Dq + k] = acc[k];
        if (j == 0)
            for (int k = 0; k < Dq; ++k) part[(size_t)Dq * Dv * Dq + (size_t)i * Dq + k] = kk[k];
    }
}

__global__ __launch_bounds__(kThreads) void triple_merge_kernel(TripleArgs a)
{
    const size_t ns = (size_t)a.Dq * a.Dv * a.Dq, nk = (size_t)a.Dq * a.Dq;
    const size_t per = triple_partial_floats(a.Dq, a.Dv, a.diag_parts != 0);
    const size_t total = (size_t)a.B * a.H * per;
    const size_t idx = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const size_t bh = idx / per, e = idx - bh * per;
    const float* p = a.part + bh * a.n_parts * per + e;
    // eight partials requested at a time (a load per iteration would wait for the one before); summed in split order
    float s = 0.f;
    for (int sp = 0; sp < a.n_parts; sp += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = p[(size_t)min(sp + u, a.n_parts - 1) * per];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += sp + u < a.n_parts ? t[u] : 0.f;
    }
    s *= 1.0f / (float)a.N;
    if (!a.diag_parts) {
        if (e < ns) a.state[bh * ns + e] = s;
        else if (a.kk) a.kk[bh * nk + (e - ns)] = s;
        return;
    }
    // Matrix-core partials: one 16 x 16 x 16 block after the other, each in the kernel's accumulator order.  Element
    // (step r, lane = 16 g + c16, register rr) of a block holds state[i = 4g + rr][j = c16][k = (i - r) mod 16] of
    // the block; the tile behind the sixteen steps holds the block's kk[i = 4g + rr][k' = c16] (the same for every
    // column block jb: taken from jb = 0).
    const int nbq = a.Dq >> 4, nbv = a.Dv >> 4;
    const int blk = (int)(e / 4352), o = (int)(e % 4352);
    const int ib = blk / (nbv * nbq), jb = (blk / nbq) % nbv, kb = blk % nbq;
    const int r = o >> 8, lane = (o >> 2) & 63, rr = o & 3;
    const int i = 4 * (lane >> 4) + rr, c16 = lane & 15;
    if (o < 4096) {
        a.state[bh * ns + ((size_t)(16 * ib + i) * a.Dv + 16 * jb + c16) * a.Dq + 16 * kb + ((i - r) & 15)] = s;
    } else if (a.kk && jb == 0) {
        a.kk[bh * nk + (size_t)(16 * ib + i) * a.Dq + 16 * kb + c16] = s;
    }
}

constexpr int kOutLdsFloats = 8192;

// One thread per token; state rows staged through LDS IB rows at a time (broadcast reads).
template <typename T, int DQ, int DV>
__global__ __launch_bounds__(kThreads) void triple_out_kernel(TripleArgs a)
{
    __shared__ float st[kOutLdsFloats];
    __shared__ float kks[DQ * DQ];

    const int tid = threadIdx.x;
    const int Dq = a.Dq, Dv = a.Dv;
    const int h = blockIdx.y, b = blockIdx.z;
    const int n = blockIdx.x * kThreads + tid;
    const bool live = n < a.N;
    const size_t bh = (size_t)b * a.H + h;

    const T* q1 = (const T*)a.q1 + b * a.q1s[0] + h * a.q1s[1];
    const T* q2 = (const T*)a.q2 + b * a.q2s[0] + h * a.q2s[1];
    const float* state = a.state + bh * Dq * Dv * Dq;

    float r1[DQ], r2[DQ], out[DV];
#pragma unroll
    for (int d = 0; d < DQ; ++d) {
        r1[d] = (live && d < Dq) ? feat(to_f32(q1[(int64_t)n * a.q1s[2] + d]), a.feature_map) : 0.f;
        r2[d] = (live && d < Dq) ? feat(to_f32(q2[(int64_t)n * a.q2s[2] + d]), a.feature_map) : 0.f;
    }
#pragma unroll
    for (int jj = 0; jj < DV; ++jj) out[jj] = 0.f;

    float den = 1.f;
    if (a.normalize) {
        for (int idx = tid; idx < Dq * Dq; idx += kThreads) kks[idx] = a.kk[bh * Dq * Dq + idx];
        __syncthreads();
        den = 0.f;
#pragma unroll
        for (int i = 0; i < DQ; ++i) {
            if (i < Dq) {
                float t = 0.f;
#pragma unroll
                for (int k = 0; k < DQ; ++k)
                    if (k < Dq) t = fmaf(kks[i * Dq + k], r2[k], t);
                den = fmaf(r1[i], t, den);
            }
        }
    }

    const int rowf = Dv * Dq;               // floats per state row i
    const int IB = max(1, kOutLdsFloats / rowf);
    for (int i0 = 0; i0 < Dq; i0 += IB) {
        const int ib = min(IB, Dq - i0);
        __syncthreads();
        for (int idx = tid; idx < ib * rowf; idx += kThreads) st[idx] = state[(size_t)i0 * rowf + idx];
        __syncthreads();
        for (int il = 0; il < ib; ++il) {
            float qi = 0.f;
#pragma unroll
            for (int d = 0; d < DQ; ++d)
                if (d == i0 + il) qi = r1[d];
#pragma unroll
            for (int jj = 0; jj < DV; ++jj) {
                if (jj < Dv) {
                    float t = 0.f;
#pragma unroll
                    for (int k = 0; k < DQ; ++k)
                        if (k < Dq) t = fmaf(st[(il * Dv + jj) * Dq + k], r2[k], t);
                    out[jj] = fmaf(qi, t, out[jj]);
                }
            }
        }
    }
    if (live) {
        const float inv = a.normalize ? 1.f / den : 1.f;
        T* o = (T*)a.out + b * a.os[0] + h * a.os[1] + (int64_t)n * a.os[2];
#pragma unroll
        for (int jj = 0; jj < DV; ++jj)
            if (jj < Dv) o[jj] = from_f32<T>(out[jj] * inv);
    }
}

template <typename T>
hipError_t state_launch(const TripleArgs& a, hipStream_t st)
{
    int IB = kThreads / a.Dv;
    if (IB < 1) IB = 1;
    if (IB > a.Dq) IB = a.Dq;
    const int iblocks = (a.Dq + IB - 1) / IB;
    dim3 grid(a.n_splits * iblocks, a.H, a.B);
    if (a.Dq <= 16)      hipLaunchKernelGGL((triple_state_kernel<T, 16>), grid, dim3(kThreads), 0, st, a, IB);
    else if (a.Dq <= 32) hipLaunchKernelGGL((triple_state_kernel<T, 32>), grid, dim3(kThreads), 0, st, a, IB);
    else                 hipLaunchKernelGGL((triple_state_kernel<T, 64>), grid, dim3(kThreads), 0, st, a, IB);
    return hipGetLastError();
}

template <typename T>
hipError_t out_launch(const TripleArgs& a, hipStream_t st)
{
    dim3 grid((a.N + kThreads - 1) / kThreads, a.H, a.B);
    const int dm = a.Dq > a.Dv ? a.Dq : a.Dv;
    if (dm <= 16)      hipLaunchKernelGGL((triple_out_kernel<T, 16, 16>), grid, dim3(kThreads), 0, st, a);
    else if (dm <= 32) hipLaunchKernelGGL((triple_out_kernel<T, 32, 32>), grid, dim3(kThreads), 0, st, a);
    else               hipLaunchKernelGGL((triple_out_kernel<T, 64, 64>), grid, dim3(kThreads), 0, st, a);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_triple_state(const TripleArgs& a, int dtype, hipStream_t st)
{
    if (dtype == 0 && triple_f32_mfma_state_ok(a)) return launch_triple_state_f32_mfma(a, st);     // fp32, head dims 16
    switch (dtype) {
        case 0: return state_launch<float>(a, st);
        case 1: return state_launch<bf16_t>(a, st);
        default: return state_launch<f16_t>(a, st);
    }
}

hipError_t launch_triple_merge(const TripleArgs& a, hipStream_t st)
{
    const size_t per = triple_partial_floats(a.Dq, a.Dv, a.diag_parts != 0);
    const size_t total = (size_t)a.B * a.H * per;
    hipLaunchKernelGGL(triple_merge_kernel, dim3((unsigned)((total + kThreads - 1) / kThreads)), dim3(kThreads), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_triple_out(const TripleArgs& a, int dtype, hipStream_t st)
{
    if (dtype == 0 && triple_f32_mfma_out_ok(a)) return launch_triple_out_f32_mfma(a, st);
    switch (dtype) {
        case 0: return out_launch<float>(a, st);
        case 1: return out_launch<bf16_t>(a, st);
        default: return out_launch<f16_t>(a, st);
    }
}

}  // namespace flare
