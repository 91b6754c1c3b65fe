// Generic (any M, D <= 128, any dtype, strided, masked) FLARE mixer kernels.
//
// All arithmetic is fp32 FMA with exp2 on log2-scaled scores; these kernels are the fp32
// parity path and the fallback for shapes the MFMA kernels do not cover.  They share the
// split-N partial format and the merge kernel with the MFMA gather.
//
//   gather : z[b,h,m,:] = sum_n softmax_n(s <q_m,k_n>) v_n        (README.md:49 of the reference)
//   scatter: y[b,h,n,:] = sum_m softmax_m(s <k_n,q_m>) z_m        (README.md:50)
#include "common.hpp"

namespace flare {

namespace {

constexpr int kGatherThreads = 256;
constexpr int kGatherLat     = 64;   // latents per workgroup (one per lane)
constexpr int kGatherGroups  = 4;    // token groups per workgroup (one per wave)
constexpr int kGatherTile    = 32;   // tokens staged in LDS per iteration

// One workgroup: 64 latents x one contiguous token range.  Lane = latent, wave = token
// group; every wave keeps its own online-softmax partial and writes it out as a separate
// partial, so no cross-wave combine is needed and the merge order is fixed.
template <typename T, int DMAX>
__global__ __launch_bounds__(kGatherThreads) void gather_generic_kernel(MixerArgs a)
{
    __shared__ float ks[kGatherTile][DMAX];
    __shared__ float vs[kGatherTile][DMAX];
    __shared__ int   keep[kGatherTile];

    const int tid = threadIdx.x;
    const int ml = tid & 63, g = tid >> 6;
    const int mblocks = (a.M + kGatherLat - 1) / kGatherLat;
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;
    const int m = mb * kGatherLat + ml;
    const int D = a.D;

    const T* q = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
    const T* k = (const T*)a.k + b * a.ks[0] + h * a.ks[1];
    const T* v = (const T*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint8_t* mask = a.mask ? a.mask + (int64_t)b * a.N : nullptr;

    float qr[DMAX], acc[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
        qr[d] = (m < a.M && d < D) ? to_f32(q[m * a.qs[2] + d]) * a.scale_log2 : 0.f;
        acc[d] = 0.f;
    }
    float mx = kNegBig, l = 0.f;
    const uint32_t bh = (uint32_t)(b * a.H + h);

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);

    for (int n0 = n_begin; n0 < n_end; n0 += kGatherTile) {
        const int tn = min(kGatherTile, n_end - n0);
        __syncthreads();
        for (int idx = tid; idx < tn * D; idx += kGatherThreads) {
            const int j = idx / D, d = idx - j * D;
            ks[j][d] = to_f32(k[(int64_t)(n0 + j) * a.ks[2] + d]);
            vs[j][d] = to_f32(v[(int64_t)(n0 + j) * a.vs[2] + d]);
        }
        if (tid < tn) keep[tid] = mask ? (int)mask[n0 + tid] : 1;
        __syncthreads();
        for (int j = g; j < tn; j += kGatherGroups) {
            if (!keep[j]) continue;
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < DMAX; ++d)
                if (d < D) s = fmaf(qr[d], ks[j][d], s);
            const float mn = fmaxf(mx, s);
            const float al = fast_exp2(mx - mn);
            const float p = fast_exp2(s - mn);
            l = l * al + p;
            // dropout acts on the normalised weight: the denominator keeps every term, the numerator the kept ones
            float pv = p;
            if (a.drop_thr != 0)
                pv = dropout_hash24(a.seed_lo, a.seed_hi, 0u, bh, (uint32_t)m, (uint32_t)(n0 + j)) >= a.drop_thr ? p * a.drop_rs : 0.f;
#pragma unroll
            for (int d = 0; d < DMAX; ++d)
                if (d < D) acc[d] = fmaf(acc[d], al, pv * vs[j][d]);
            mx = mn;
        }
    }

    if (m < a.M) {
        const int part = split * kGatherGroups + g;
        const int64_t row = (((int64_t)b * a.H + h) * a.n_parts + part) * a.M + m;
        a.part_m[row] = mx;
        a.part_l[row] = l;
        for (int d = 0; d < D; ++d) a.part_acc[row * D + d] = acc[d];
    }
}

// Fixed-order merge of the split-N partials: bit-stable for a given n_parts.
// One thread per (b,h,m,d); partials are visited in batches of 8 so that the loads of a batch
// are all in flight before the first is consumed.
__global__ __launch_bounds__(256) void gather_merge_kernel(MixerArgs a)
{
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)a.B * a.H * a.M * a.D;
    if (idx >= total) return;
    const int d = idx % a.D;
    const int64_t r = idx / a.D;          // (b*H + h)*M + m
    const int m = r % a.M;
    const int64_t bh = r / a.M;
    const int P = a.n_parts;
    const float* __restrict__ pm = a.part_m + bh * P * a.M + m;
    const float* __restrict__ pl = a.part_l + bh * P * a.M + m;
    const float* __restrict__ pa = a.part_acc + (bh * P * a.M + m) * a.D + d;
    const int64_t sm = a.M, sa = (int64_t)a.M * a.D;
    constexpr int U = 8;

    float mx = kNegBig;
    int p = 0;
    for (; p + U <= P; p += U) {
        float t[U];
#pragma unroll
        for (int u = 0; u < U; ++u) t[u] = pm[(p + u) * sm];
#pragma unroll
        for (int u = 0; u < U; ++u) mx = fmaxf(mx, t[u]);
    }
    for (; p < P; ++p) mx = fmaxf(mx, pm[p * sm]);

    float l = 0.f, acc = 0.f;
    p = 0;
    for (; p + U <= P; p += U) {
        float tm[U], tl[U], ta[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            tm[u] = pm[(p + u) * sm];
            tl[u] = pl[(p + u) * sm];
            ta[u] = pa[(p + u) * sa];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float w = fast_exp2(tm[u] - mx);
            l = fmaf(tl[u], w, l);
            acc = fmaf(ta[u], w, acc);
        }
    }
    for (; p < P; ++p) {
        const float w = fast_exp2(pm[p * sm] - mx);
        l = fmaf(pl[p * sm], w, l);
        acc = fmaf(pa[p * sa], w, acc);
    }
    a.z[idx] = l > 0.f ? acc / l : 0.f;
    if (a.lse && d == 0) a.lse[r] = l > 0.f ? (mx + __log2f(l)) * kLn2 : -INFINITY;
}

constexpr int kScatterThreads = 256;
constexpr int kScatterLdsElems = 4096;  // q and z chunk: MC * DMAX floats each

// One thread per token; Q and Z staged through LDS in chunks of MC latents with an online
// softmax across chunks.  Every lane reads the same LDS address (broadcast).
template <typename T, int DMAX>
__global__ __launch_bounds__(kScatterThreads) void scatter_generic_kernel(MixerArgs a)
{
    constexpr int MC = kScatterLdsElems / DMAX;
    __shared__ float qs[MC][DMAX];
    __shared__ float zs[MC][DMAX];

    const int tid = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
    const int n = blockIdx.x * kScatterThreads + tid;
    const int D = a.D;
    const bool live = n < a.N;

    const T* q = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
    const T* k = (const T*)a.k + b * a.ks[0] + h * a.ks[1];
    const float* z = a.z + ((int64_t)b * a.H + h) * a.M * D;

    float kr[DMAX], acc[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
        kr[d] = (live && d < D) ? to_f32(k[(int64_t)n * a.ks[2] + d]) * a.scale_log2 : 0.f;
        acc[d] = 0.f;
    }
    float mx = kNegBig, l = 0.f;

    for (int m0 = 0; m0 < a.M; m0 += MC) {
        const int mc = min(MC, a.M - m0);
        __syncthreads();
        for (int idx = tid; idx < mc * D; idx += kScatterThreads) {
            const int j = idx / D, d = idx - j * D;
            qs[j][d] = to_f32(q[(int64_t)(m0 + j) * a.qs[2] + d]);
            zs[j][d] = z[(int64_t)(m0 + j) * D + d];
        }
        __syncthreads();
        for (int j = 0; j < mc; ++j) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < DMAX; ++d)
                if (d < D) s = fmaf(kr[d], qs[j][d], s);
            const float mn = fmaxf(mx, s);
            const float al = fast_exp2(mx - mn);
            const float p = fast_exp2(s - mn);
            l = l * al + p;
            float pv = p;
            if (a.drop_thr != 0)
                pv = dropout_hash24(a.seed_lo, a.seed_hi, 1u, (uint32_t)(b * a.H + h), (uint32_t)(m0 + j), (uint32_t)n) >= a.drop_thr
                         ? p * a.drop_rs : 0.f;
#pragma unroll
            for (int d = 0; d < DMAX; ++d)
                if (d < D) acc[d] = fmaf(acc[d], al, pv * zs[j][d]);
            mx = mn;
        }
    }

    if (live) {
        const bool on = a.mask ? a.mask[(int64_t)b * a.N + n] != 0 : true;
        const float inv = on ? 1.f / l : 0.f;
        if (a.lse_tok) a.lse_tok[((int64_t)b * a.H + h) * a.N + n] = (mx + __log2f(l)) * kLn2;
        T* y = (T*)a.y + b * a.ys[0] + h * a.ys[1] + (int64_t)n * a.ys[2];
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < D) y[d] = from_f32<T>(on ? acc[d] * inv : 0.f);      // a padded row is 0 whatever its key row held
    }
}

template <typename T>
hipError_t gather_dispatch_d(const MixerArgs& a, dim3 grid, hipStream_t st)
{
    if (a.D <= 16)       hipLaunchKernelGGL((gather_generic_kernel<T, 16>), grid, dim3(kGatherThreads), 0, st, a);
    else if (a.D <= 32)  hipLaunchKernelGGL((gather_generic_kernel<T, 32>), grid, dim3(kGatherThreads), 0, st, a);
    else if (a.D <= 64)  hipLaunchKernelGGL((gather_generic_kernel<T, 64>), grid, dim3(kGatherThreads), 0, st, a);
    else                 hipLaunchKernelGGL((gather_generic_kernel<T, 128>), grid, dim3(kGatherThreads), 0, st, a);
    return hipGetLastError();
}

template <typename T>
hipError_t scatter_dispatch_d(const MixerArgs& a, dim3 grid, hipStream_t st)
{
    if (a.D <= 16)       hipLaunchKernelGGL((scatter_generic_kernel<T, 16>), grid, dim3(kScatterThreads), 0, st, a);
    else if (a.D <= 32)  hipLaunchKernelGGL((scatter_generic_kernel<T, 32>), grid, dim3(kScatterThreads), 0, st, a);
    else if (a.D <= 64)  hipLaunchKernelGGL((scatter_generic_kernel<T, 64>), grid, dim3(kScatterThreads), 0, st, a);
    else                 hipLaunchKernelGGL((scatter_generic_kernel<T, 128>), grid, dim3(kScatterThreads), 0, st, a);
    return hipGetLastError();
}

}  // namespace

int gather_generic_parts_per_wg() { return kGatherGroups; }

hipError_t launch_gather_generic(const MixerArgs& a, int dtype, hipStream_t st)
{
    // fp32 problems the matrix-core kernels take (same grid, one partial per wave as here)
    if (dtype == 0 && f32_mfma_mixer_ok(a, false)) return launch_gather_f32_mfma(a, st);
    const int mblocks = (a.M + kGatherLat - 1) / kGatherLat;
    dim3 grid(a.n_splits * mblocks, a.H, a.B);
    switch (dtype) {
        case 0: return gather_dispatch_d<float>(a, grid, st);
        case 1: return gather_dispatch_d<bf16_t>(a, grid, st);
        default: return gather_dispatch_d<f16_t>(a, grid, st);
    }
}

hipError_t launch_gather_merge(const MixerArgs& a, hipStream_t st)
{
    const int64_t total = (int64_t)a.B * a.H * a.M * a.D;
    dim3 grid((unsigned)((total + 255) / 256));
    hipLaunchKernelGGL(gather_merge_kernel, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_scatter_generic(const MixerArgs& a, int dtype, hipStream_t st)
{
    if (dtype == 0 && f32_mfma_mixer_ok(a, true)) return launch_scatter_f32_mfma(a, st);
    dim3 grid((a.N + kScatterThreads - 1) / kScatterThreads, a.H, a.B);
    switch (dtype) {
        case 0: return scatter_dispatch_d<float>(a, grid, st);
        case 1: return scatter_dispatch_d<bf16_t>(a, grid, st);
        default: return scatter_dispatch_d<f16_t>(a, grid, st);
    }
}

}  // namespace flare
