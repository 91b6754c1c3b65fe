// Triple (third-order) linear attention for fp32 inputs with head dims 16 or 32 on v_mfma_f32_16x16x4_f32
// (lra/models/backends.py:1285-1292, lra/models/triton/triple.py:29-121 of the reference):
//   state[i,j,k] = (1/N) sum_n f(k1)[n,i] v[n,j] f(k2)[n,k],   out[n,j] = sum_{i,k} f(q1)[n,i] state[i,j,k] f(q2)[n,k].
// Taken by the fp32 launchers of triple.hip when Dq = Dv = 16 or 32 and the rows are 16-byte aligned; same split-N partials
// ([i][j][k] and the normaliser's [i][k]), merge kernel and workspace layout as the FMA kernels there.
//
// The instruction takes one float per lane for A (row c16, k-slot = lane group g) and for B (column c16, k-slot g).
// State: for every i a 16 x 16 tile over (k, j), contracted over four tokens at a time: A = f(k1)[n,i] f(k2)[n,k]
// (f(k1)[n,i] by a shuffle from the lane that holds it, one multiply per lane and instruction), B = v[n,j].  Output: out^T[j, n] contracted over the 256 pairs (i,k), four k
// at a time: A = state[i][j][k] from LDS, B = f(q1)[n,i] f(q2)[n,k] (one multiply again).  The normaliser rides along
// as plain sums of the same products.
#include <algorithm>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mma4(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
__device__ __forceinline__ float feat(float x, int fm)
{
    if (!fm) return x;
    return x > 0.f ? x + 1.f : __expf(x);
}
__device__ __forceinline__ float groups_sum(float x)
{
    x += __shfl_xor(x, 16);
    return x + __shfl_xor(x, 32);
}

constexpr int kD = 16;

// grid = (n_splits, H, B).  Wave w takes the 16-token groups w, w + 4, ... of the split; the four waves' sums meet in
// LDS in wave order (bit-stable) and wave 0 writes the split's partial.
__global__ __launch_bounds__(256, 2) void triple_state_f32_mfma_kernel(TripleArgs a)
{
    __shared__ __attribute__((aligned(16))) f32x4 red[3][kD][64];
    __shared__ float redk[3][kD][64];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const float* k1 = (const float*)a.k1 + b * a.k1s[0] + h * a.k1s[1];
    const float* k2 = (const float*)a.k2 + b * a.k2s[0] + h * a.k2s[1];
    const float* v = (const float*)a.v + b * a.vs[0] + h * a.vs[1];

    f32x4 acc[kD];
    float kkacc[kD];
#pragma unroll
    for (int i = 0; i < kD; ++i) {
        acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        kkacc[i] = 0.f;
    }
    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int groups = n_begin < n_end ? (n_end - n_begin + 15) / 16 : 0;
    const int mine = groups > w ? (groups - w + 3) / 4 : 0;

    // the lane's four tokens of a group are 4c + g, c = 0..3: feature c16 of their k1, k2 and v rows.  f(k1)[n, i] for
    // the other i comes from the lane (g, i) by a shuffle: one feature map per lane and token instead of sixteen.
    // The next group is requested while this one is worked on (rows past the split repeat its last row, no branch).
    float k1n[4], k2n[4], vn[4];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int n = max(min(n0 + 4 * c + g, n_end - 1), 0);
            k1n[c] = k1[(int64_t)n * a.k1s[2] + c16];
            k2n[c] = k2[(int64_t)n * a.k2s[2] + c16];
            vn[c] = v[(int64_t)n * a.vs[2] + c16];
        }
    };
    int n0 = n_begin + 16 * w;
    if (mine > 0) fetch(n0);
    for (int t = 0; t < mine; ++t, n0 += 64) {
        float k1c[4], k2c[4], vc[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const bool valid = n0 + 4 * c + g < n_end;
            k1c[c] = feat(k1n[c], a.feature_map);
            k2c[c] = valid ? feat(k2n[c], a.feature_map) : 0.f;       // a token past the split adds nothing
            vc[c] = valid ? vn[c] : 0.f;
        }
        fetch(n0 + 64);
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int i = 0; i < kD; ++i) {
                const float p = __shfl(k1c[c], (lane & 48) | i) * k2c[c];
                acc[i] = mma4(p, vc[c], acc[i]);        // rows k = 4g + r, column j = c16
                kkacc[i] += p;                          // kk[i][k = c16], this lane group's tokens
            }
    }

    if (w > 0) {
#pragma unroll
        for (int i = 0; i < kD; ++i) {
            red[w - 1][i][lane] = acc[i];
            redk[w - 1][i][lane] = kkacc[i];
        }
    }
    __syncthreads();
    if (w > 0) return;
    constexpr size_t per = (size_t)kD * kD * kD + (size_t)kD * kD;
    float* part = a.part + (((size_t)b * a.H + h) * a.n_parts + split) * per;
#pragma unroll
    for (int i = 0; i < kD; ++i) {
        f32x4 s = acc[i];
        float kk = kkacc[i];
#pragma unroll
        for (int ww = 0; ww < 3; ++ww) {
            s += red[ww][i][lane];
            kk += redk[ww][i][lane];
        }
        kk = groups_sum(kk);
        *reinterpret_cast<f32x4*>(part + ((size_t)i * kD + c16) * kD + 4 * g) = s;      // [i][j = c16][k = 4g + r]
        if (g == 0) part[(size_t)kD * kD * kD + (size_t)i * kD + c16] = kk;
    }
}

// grid = (workgroups, H, B); a wave takes 16 tokens at a time.
__global__ __launch_bounds__(256) void triple_out_f32_mfma_kernel(TripleArgs a)
{
    __shared__ float ss[kD * kD * 17];      // state[i][j][k] at (i 16 + j) 17 + k: the 16 rows j of a read fall into 16 banks
    __shared__ float kks[kD * kD];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const float* q1 = (const float*)a.q1 + b * a.q1s[0] + h * a.q1s[1];
    const float* q2 = (const float*)a.q2 + b * a.q2s[0] + h * a.q2s[1];
    float* out = (float*)a.out + b * a.os[0] + h * a.os[1];
    const float* state = a.state + bh * kD * kD * kD;

    for (int idx = tid; idx < kD * kD * kD; idx += 256) ss[(idx >> 4) * 17 + (idx & 15)] = state[idx];
    if (a.normalize) kks[tid] = a.kk[bh * kD * kD + tid];
    __syncthreads();

    const int tiles = (a.N + 15) / 16, stride = gridDim.x * 4;
    int tile = blockIdx.x * 4 + w;
    const int mine = tile < tiles ? (tiles - tile + stride - 1) / stride : 0;
    f32x4 q1n[4];
    float q2n[4];
    auto fetch = [&](int tl) {
        const int n = min(tl * 16 + c16, a.N - 1);
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) q1n[q4] = *reinterpret_cast<const f32x4*>(q1 + (int64_t)n * a.q1s[2] + 4 * q4);
#pragma unroll
        for (int kq = 0; kq < 4; ++kq) q2n[kq] = q2[(int64_t)n * a.q2s[2] + 4 * kq + g];
    };
    if (mine > 0) fetch(tile);
    for (int t = 0; t < mine; ++t, tile += stride) {
        float q1c[kD], q2c[4];
#pragma unroll
        for (int i = 0; i < kD; ++i) q1c[i] = feat(q1n[i >> 2][i & 3], a.feature_map);
#pragma unroll
        for (int kq = 0; kq < 4; ++kq) q2c[kq] = feat(q2n[kq], a.feature_map);
        fetch(tile + stride);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        float den = 0.f;
#pragma unroll
        for (int i = 0; i < kD; ++i)
#pragma unroll
            for (int kq = 0; kq < 4; ++kq) {
                const float p = q1c[i] * q2c[kq];                                   // token c16, pair (i, k = 4 kq + g)
                acc = mma4(ss[(i * kD + c16) * 17 + 4 * kq + g], p, acc);           // rows j = 4g + r, column n = c16
                if (a.normalize) den = fmaf(p, kks[i * kD + 4 * kq + g], den);
            }
        den = a.normalize ? groups_sum(den) : 1.f;
        const int n = tile * 16 + c16;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the next tile's rows, before the stores
        if (n < a.N) *reinterpret_cast<f32x4*>(out + (int64_t)n * a.os[2] + 4 * g) = acc * (1.f / den);
    }
}

// ---- head dims 32: the same scheme with 2 x 2 tiles over (k, j) per i -------------------------------------------
// State: grid = (n_splits * 4, H, B), a workgroup owns eight rows i of the state (32 accumulator tiles per wave).
__global__ __launch_bounds__(256, 2) void triple_state_f32_mfma32_kernel(TripleArgs a)
{
    constexpr int D = 32, IB = 8;
    __shared__ __attribute__((aligned(16))) f32x4 red[IB * 4][64];
    __shared__ float redk[IB * 2][64];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int split = blockIdx.x >> 2, i0 = (blockIdx.x & 3) * IB, h = blockIdx.y, b = blockIdx.z;
    const float* k1 = (const float*)a.k1 + b * a.k1s[0] + h * a.k1s[1];
    const float* k2 = (const float*)a.k2 + b * a.k2s[0] + h * a.k2s[1];
    const float* v = (const float*)a.v + b * a.vs[0] + h * a.vs[1];

    f32x4 acc[IB][2][2];      // [i][k tile][j tile]: rows k = 16 kt + 4g + r, column j = 16 jt + c16
    float kkacc[IB][2];
#pragma unroll
    for (int il = 0; il < IB; ++il)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            kkacc[il][kt] = 0.f;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) acc[il][kt][jt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int groups = n_begin < n_end ? (n_end - n_begin + 15) / 16 : 0;
    const int mine = groups > w ? (groups - w + 3) / 4 : 0;

    // the lane's four tokens of a group are 4c + g; it holds f(k1)[n][i0 + (c16 & 7)] (handed round by shuffles),
    // features c16 and 16 + c16 of k2 and of v
    float k1n[4], k2n[4][2], vn[4][2];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int n = max(min(n0 + 4 * c + g, n_end - 1), 0);
            k1n[c] = k1[(int64_t)n * a.k1s[2] + i0 + (c16 & 7)];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                k2n[c][t] = k2[(int64_t)n * a.k2s[2] + 16 * t + c16];
                vn[c][t] = v[(int64_t)n * a.vs[2] + 16 * t + c16];
            }
        }
    };
    int n0 = n_begin + 16 * w;
    if (mine > 0) fetch(n0);
    for (int t = 0; t < mine; ++t, n0 += 64) {
        float k1c[4], k2c[4][2], vc[4][2];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const bool valid = n0 + 4 * c + g < n_end;
            k1c[c] = feat(k1n[c], a.feature_map);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                k2c[c][u] = valid ? feat(k2n[c][u], a.feature_map) : 0.f;
                vc[c][u] = valid ? vn[c][u] : 0.f;
            }
        }
        fetch(n0 + 64);
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int il = 0; il < IB; ++il) {
                const float kf = __shfl(k1c[c], (lane & 48) | il);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    const float p = kf * k2c[c][kt];
                    kkacc[il][kt] += p;
#pragma unroll
                    for (int jt = 0; jt < 2; ++jt) acc[il][kt][jt] = mma4(p, vc[c][jt], acc[il][kt][jt]);
                }
            }
    }

    // waves 1..3 hand their sums to wave 0 one after the other (fixed order)
    for (int ww = 1; ww < 4; ++ww) {
        if (w == ww) {
#pragma unroll
            for (int il = 0; il < IB; ++il)
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    redk[il * 2 + kt][lane] = kkacc[il][kt];
#pragma unroll
                    for (int jt = 0; jt < 2; ++jt) red[(il * 2 + kt) * 2 + jt][lane] = acc[il][kt][jt];
                }
        }
        __syncthreads();
        if (w == 0) {
#pragma unroll
            for (int il = 0; il < IB; ++il)
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    kkacc[il][kt] += redk[il * 2 + kt][lane];
#pragma unroll
                    for (int jt = 0; jt < 2; ++jt) acc[il][kt][jt] += red[(il * 2 + kt) * 2 + jt][lane];
                }
        }
        __syncthreads();
    }
    if (w > 0) return;
    constexpr size_t per = (size_t)D * D * D + (size_t)D * D;
    float* part = a.part + (((size_t)b * a.H + h) * a.n_parts + split) * per;
#pragma unroll
    for (int il = 0; il < IB; ++il)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const float kk = groups_sum(kkacc[il][kt]);
            if (g == 0) part[(size_t)D * D * D + (size_t)(i0 + il) * D + 16 * kt + c16] = kk;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
                *reinterpret_cast<f32x4*>(part + ((size_t)(i0 + il) * D + 16 * jt + c16) * D + 16 * kt + 4 * g) = acc[il][kt][jt];
        }
}

// Output: all of the (b,h)'s state in LDS (rows padded to 33 floats), eight waves, 16 tokens per wave and pass.
__global__ __launch_bounds__(512) void triple_out_f32_mfma32_kernel(TripleArgs a)
{
    constexpr int D = 32;
    extern __shared__ __attribute__((aligned(16))) float smem_t[];
    float* ss = smem_t;                       // state[i][j][k] at (i 32 + j) 33 + k
    float* kks = smem_t + D * D * 33;         // kk[i][k]

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const float* q1 = (const float*)a.q1 + b * a.q1s[0] + h * a.q1s[1];
    const float* q2 = (const float*)a.q2 + b * a.q2s[0] + h * a.q2s[1];
    float* out = (float*)a.out + b * a.os[0] + h * a.os[1];
    const float* state = a.state + bh * D * D * D;

    for (int idx = tid; idx < D * D * D; idx += 512) ss[(idx >> 5) * 33 + (idx & 31)] = state[idx];
    if (a.normalize)
        for (int idx = tid; idx < D * D; idx += 512) kks[idx] = a.kk[bh * D * D + idx];
    __syncthreads();

    const int tiles = (a.N + 15) / 16, stride = gridDim.x * 8;
    int tile = blockIdx.x * 8 + w;
    const int mine = tile < tiles ? (tiles - tile + stride - 1) / stride : 0;
    f32x4 q1n[8];
    float q2n[8];
    auto fetch = [&](int tl) {
        const int n = min(tl * 16 + c16, a.N - 1);
#pragma unroll
        for (int q4 = 0; q4 < 8; ++q4) q1n[q4] = *reinterpret_cast<const f32x4*>(q1 + (int64_t)n * a.q1s[2] + 4 * q4);
#pragma unroll
        for (int kq = 0; kq < 8; ++kq) q2n[kq] = q2[(int64_t)n * a.q2s[2] + 4 * kq + g];
    };
    if (mine > 0) fetch(tile);
    for (int t = 0; t < mine; ++t, tile += stride) {
        float q1c[D], q2c[8];
#pragma unroll
        for (int i = 0; i < D; ++i) q1c[i] = feat(q1n[i >> 2][i & 3], a.feature_map);
#pragma unroll
        for (int kq = 0; kq < 8; ++kq) q2c[kq] = feat(q2n[kq], a.feature_map);
        fetch(tile + stride);
        f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
        float den = 0.f;
#pragma unroll
        for (int i = 0; i < D; ++i)
#pragma unroll
            for (int kq = 0; kq < 8; ++kq) {
                const float p = q1c[i] * q2c[kq];                                   // token c16, pair (i, k = 4 kq + g)
#pragma unroll
                for (int jt = 0; jt < 2; ++jt) acc[jt] = mma4(ss[(i * D + 16 * jt + c16) * 33 + 4 * kq + g], p, acc[jt]);
                if (a.normalize) den = fmaf(p, kks[i * D + 4 * kq + g], den);
            }
        den = a.normalize ? groups_sum(den) : 1.f;
        const int n = tile * 16 + c16;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the next tile's rows, before the stores
        if (n < a.N) {
            const float inv = 1.f / den;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) *reinterpret_cast<f32x4*>(out + (int64_t)n * a.os[2] + 16 * jt + 4 * g) = acc[jt] * inv;
        }
    }
}

bool rows16(const void* p, const int64_t* s)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && s[0] % 4 == 0 && s[1] % 4 == 0 && s[2] % 4 == 0;
}

}  // namespace

bool triple_f32_mfma_state_ok(const TripleArgs& a)
{
    return a.Dq == a.Dv && (a.Dq == 16 || a.Dq == 32) && !a.diag_parts && (reinterpret_cast<uintptr_t>(a.part) & 15) == 0;
}

bool triple_f32_mfma_out_ok(const TripleArgs& a)
{
    return a.Dq == a.Dv && (a.Dq == 16 || a.Dq == 32) && rows16(a.q1, a.q1s) && rows16(a.q2, a.q2s) && rows16(a.out, a.os);
}

hipError_t launch_triple_state_f32_mfma(const TripleArgs& a, hipStream_t st)
{
    if (a.Dq == 32) hipLaunchKernelGGL(triple_state_f32_mfma32_kernel, dim3(a.n_splits * 4, a.H, a.B), dim3(256), 0, st, a);
    else            hipLaunchKernelGGL(triple_state_f32_mfma_kernel, dim3(a.n_splits, a.H, a.B), dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_triple_out_f32_mfma(const TripleArgs& a, hipStream_t st)
{
    const int64_t bh = (int64_t)a.B * a.H;
    if (a.Dq == 32) {
        constexpr size_t lds = (size_t)(32 * 32 * 33 + 32 * 32) * 4;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(triple_out_f32_mfma32_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        const int64_t groups = ((int64_t)a.N + 127) / 128;      // one workgroup per CU: each fills 139 KB of LDS once
        const int64_t want = std::max<int64_t>(1, (device_cus() + bh - 1) / bh);
        hipLaunchKernelGGL(triple_out_f32_mfma32_kernel, dim3((unsigned)std::min<int64_t>(groups, want), a.H, a.B), dim3(512), lds, st, a);
        return hipGetLastError();
    }
    const int64_t groups = ((int64_t)a.N + 63) / 64;
    const int64_t want = std::max<int64_t>(1, ((int64_t)8 * device_cus() + bh - 1) / bh);
    hipLaunchKernelGGL(triple_out_f32_mfma_kernel, dim3((unsigned)std::min<int64_t>(groups, want), a.H, a.B), dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace flare
