// FLARE mixer for fp32 inputs on the fp32 matrix instruction v_mfma_f32_16x16x4_f32 (README.md:39-52 of the
// reference: z = softmax_n(s q k^T) v, y = softmax_m(s k q^T) z).  Taken by the fp32 launchers of mixer_generic.hip for
// D in {16, 32, 64}, M a multiple of 16 and 16-byte aligned rows, with or without attention dropout (the keep mask is
// applied to the exponentials in registers on their way into the value product; the denominators keep every weight); same
// workspace layout, partial format and merge kernel as the FMA kernels there.
//
// Operands: A is one float per lane (row c16, k = lane group g), B one float per lane (column c16, k = g), the
// accumulator lane = column c16 with rows 4g .. 4g + 3.  A product over D takes D/4 instructions; the k-slot of lane
// group g in instruction j is feature g D/4 + j, so that a lane's share of a row is contiguous in memory.  A score tile
// comes out with the softmax axis in the registers and lane groups, so its exponentials are, register r at a time, the
// B operands of the four instructions of the value product whose k-slots are the rows 4g + r: no transposition.
// Both kernels keep an exact running maximum (per latent in the gather, per token in the scatter).
#include <algorithm>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mma4(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

// maximum / sum over the four lane groups that share a column
__device__ __forceinline__ float groups_max(float x)
{
    x = fmaxf(x, __shfl_xor(x, 16));
    return fmaxf(x, __shfl_xor(x, 32));
}
__device__ __forceinline__ float groups_sum(float x)
{
    x += __shfl_xor(x, 16);
    return x + __shfl_xor(x, 32);
}

// ---- gather: one workgroup = 64 latents x one token range; wave w takes the 16-token tiles w, w + 4, ... of the range
// and writes its own partial (the layout the FMA gather uses: one partial per wave).
template <int D, bool DROP>
__global__ __launch_bounds__(256) void gather_f32_mfma_kernel(MixerArgs a)
{
    constexpr int QL = D / 4, RT = D / 16, CT = 4, VS = D + 4, VPT = D / 16;
    __shared__ __attribute__((aligned(16))) float vt[4][16][VS];     // the wave's V tile (no other wave touches it)

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int mblocks = (a.M + 63) / 64;
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;
    const float* q = (const float*)a.q + b * a.qs[0] + h * a.qs[1];
    const float* k = (const float*)a.k + b * a.ks[0] + h * a.ks[1];
    const float* v = (const float*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint8_t* mask = a.mask ? a.mask + (int64_t)b * a.N : nullptr;

    // latent operands (B of the score product), log2-scaled; latent tiles past M hold zeros and are not stored
    f32x4 qb[CT][QL / 4];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = mb * 64 + 16 * ct + c16;
#pragma unroll
        for (int j4 = 0; j4 < QL / 4; ++j4) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(q + (int64_t)min(m, a.M - 1) * a.qs[2] + g * QL + 4 * j4);
            qb[ct][j4] = m < a.M ? t * a.scale_log2 : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float mx[CT], lsum[CT];
    f32x4 zacc[CT][RT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        mx[ct] = kNegBig;
        lsum[ct] = 0.f;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) zacc[ct][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int tiles = n_begin < n_end ? (n_end - n_begin + 15) / 16 : 0;
    const int my_tiles = tiles > w ? (tiles - w + 3) / 4 : 0;

    // K rows as A operands straight from global memory, V rows through the wave's LDS tile; the next tile is requested
    // while this one is worked on (rows past the range repeat its last row: no branch around a load)
    f32x4 ka[QL / 4], vr[VPT];
    uint8_t keep_n[4] = {1, 1, 1, 1};      // key mask of the lane's four tokens (rows 4g + r of the tile)
    // the V chunk's token takes part (else it is staged as zeros: 0 * NaN is NaN): inside the range, and its mask byte,
    // kept as loaded until the chunk is staged -- a flag computed from the byte here would wait for it, and with it,
    // in order, for the K and V rows requested around it
    bool vin[VPT];
    uint32_t vmb[VPT];
    auto fetch = [&](int n0) {
        if (mask != nullptr) {
#pragma unroll
            for (int r = 0; r < 4; ++r) keep_n[r] = mask[max(min(n0 + 4 * g + r, n_end - 1), 0)];
        }
        const int n = max(min(n0 + c16, n_end - 1), 0);
#pragma unroll
        for (int j4 = 0; j4 < QL / 4; ++j4) ka[j4] = *reinterpret_cast<const f32x4*>(k + (int64_t)n * a.ks[2] + g * QL + 4 * j4);
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = lane + 64 * i, tok = c / (D / 4), ch = c % (D / 4);
            const int nv = max(min(n0 + tok, n_end - 1), 0);
            vr[i] = *reinterpret_cast<const f32x4*>(v + (int64_t)nv * a.vs[2] + 4 * ch);
            vin[i] = n0 + tok < n_end;
            vmb[i] = mask != nullptr ? (uint32_t)mask[nv] : 1u;
        }
    };
    int n0 = n_begin + 16 * w;
    if (my_tiles > 0) fetch(n0);
    for (int t = 0; t < my_tiles; ++t, n0 += 64) {
        f32x4 kc[QL / 4];
#pragma unroll
        for (int j4 = 0; j4 < QL / 4; ++j4) kc[j4] = ka[j4];
        // The tile passes between the lanes of the wave through LDS.  To the compiler every lane is a thread of its own: it
        // may move a lane's reads of other lanes' rows across that lane's own stores unless told not to.
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = lane + 64 * i, tok = c / (D / 4), ch = c % (D / 4);
            *reinterpret_cast<f32x4*>(&vt[w][tok][4 * ch]) = (vin[i] && vmb[i] != 0) ? vr[i] : f32x4{0.f, 0.f, 0.f, 0.f};
        }
        asm volatile("" ::: "memory");
        bool valid[4];      // a token past the range or padded by the key mask takes no part
#pragma unroll
        for (int r = 0; r < 4; ++r) valid[r] = n0 + 4 * g + r < n_end && keep_n[r] != 0;
        fetch(n0 + 64);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            // scores: lane = latent column c16, rows = tokens 4g + r
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j4 = 0; j4 < QL / 4; ++j4)
#pragma unroll
                for (int e = 0; e < 4; ++e) s = mma4(kc[j4][e], qb[ct][j4][e], s);
            float tm = kNegBig;
#pragma unroll
            for (int r = 0; r < 4; ++r) tm = fmaxf(tm, valid[r] ? s[r] : kNegBig);
            const float mn = fmaxf(mx[ct], groups_max(tm));
            const float al = fast_exp2(mx[ct] - mn);
            float p[4], ps = 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r] = valid[r] ? fast_exp2(s[r] - mn) : 0.f;
                ps += p[r];
            }
            lsum[ct] = lsum[ct] * al + ps;
            mx[ct] = mn;
            if constexpr (DROP) {       // the denominator keeps every weight; the numerator meets the kept ones, rescaled
                const uint32_t m = mb * 64 + 16 * ct + c16;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    p[r] = dropout_hash24(a.seed_lo, a.seed_hi, 0u, (uint32_t)(b * a.H + h), m, (uint32_t)(n0 + 4 * g + r)) >= a.drop_thr
                               ? p[r] * a.drop_rs : 0.f;
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                f32x4 z = zacc[ct][rt] * al;
#pragma unroll
                for (int r = 0; r < 4; ++r) z = mma4(vt[w][4 * g + r][16 * rt + c16], p[r], z);    // Z^T[d, m] += V^T[d, n] P[n, m]
                zacc[ct][rt] = z;
            }
        }
    }

    const int part = split * 4 + w;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = mb * 64 + 16 * ct + c16;
        const float l = groups_sum(lsum[ct]);
        if (m >= a.M) continue;
        const int64_t row = (((int64_t)b * a.H + h) * a.n_parts + part) * a.M + m;
        if (g == 0) {
            a.part_m[row] = mx[ct];
            a.part_l[row] = l;
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) *reinterpret_cast<f32x4*>(a.part_acc + row * D + 16 * rt + 4 * g) = zacc[ct][rt];
    }
}

// ---- scatter: Q (log2-scaled) and Z of one (b,h) in LDS; a wave takes 16 tokens at a time and walks all latents.
template <int D, bool DROP>
__global__ __launch_bounds__(256) void scatter_f32_mfma_kernel(MixerArgs a)
{
    constexpr int QL = D / 4, RT = D / 16, LS = D + 4;
    extern __shared__ __attribute__((aligned(16))) float smem_f[];
    float* qs = smem_f;                  // [M][LS]
    float* zs = smem_f + (size_t)a.M * LS;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const float* q = (const float*)a.q + b * a.qs[0] + h * a.qs[1];
    const float* k = (const float*)a.k + b * a.ks[0] + h * a.ks[1];
    float* y = (float*)a.y + b * a.ys[0] + h * a.ys[1];
    const float* z = a.z + ((int64_t)b * a.H + h) * a.M * D;

    for (int c = tid; c < a.M * (D / 4); c += 256) {
        const int m = c / (D / 4), ch = c % (D / 4);
        *reinterpret_cast<f32x4*>(qs + m * LS + 4 * ch) = *reinterpret_cast<const f32x4*>(q + (int64_t)m * a.qs[2] + 4 * ch) * a.scale_log2;
        *reinterpret_cast<f32x4*>(zs + m * LS + 4 * ch) = *reinterpret_cast<const f32x4*>(z + (int64_t)m * D + 4 * ch);
    }
    __syncthreads();

    const int tiles = (a.N + 15) / 16;
    const int stride = gridDim.x * 4;
    int tile = blockIdx.x * 4 + w;
    const int my_tiles = tile < tiles ? (tiles - tile + stride - 1) / stride : 0;

    // K rows as B operands straight from global memory, one tile ahead (rows past N repeat the last row)
    f32x4 kn[QL / 4];
    auto fetch = [&](int tl) {
        const int n = min(tl * 16 + c16, a.N - 1);
#pragma unroll
        for (int j4 = 0; j4 < QL / 4; ++j4) kn[j4] = *reinterpret_cast<const f32x4*>(k + (int64_t)n * a.ks[2] + g * QL + 4 * j4);
    };
    if (my_tiles > 0) fetch(tile);
    for (int t = 0; t < my_tiles; ++t, tile += stride) {
        f32x4 kb[QL / 4];
#pragma unroll
        for (int j4 = 0; j4 < QL / 4; ++j4) kb[j4] = kn[j4];
        fetch(tile + stride);
        float mx = kNegBig, lsum = 0.f;
        f32x4 yacc[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) yacc[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int mt = 0; mt < a.M / 16; ++mt) {
            // scores: lane = token column c16, rows = latents 16 mt + 4g + r
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j4 = 0; j4 < QL / 4; ++j4) {
                const f32x4 qa = *reinterpret_cast<const f32x4*>(qs + (16 * mt + c16) * LS + g * QL + 4 * j4);
#pragma unroll
                for (int e = 0; e < 4; ++e) s = mma4(qa[e], kb[j4][e], s);
            }
            const float mn = fmaxf(mx, groups_max(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]))));
            const float al = fast_exp2(mx - mn);
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) p[r] = fast_exp2(s[r] - mn);
            lsum = lsum * al + (p[0] + p[1]) + (p[2] + p[3]);
            mx = mn;
            if constexpr (DROP) {
                const uint32_t n = (uint32_t)min(tile * 16 + c16, a.N - 1);
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    p[r] = dropout_hash24(a.seed_lo, a.seed_hi, 1u, (uint32_t)(b * a.H + h), (uint32_t)(16 * mt + 4 * g + r), n) >= a.drop_thr
                               ? p[r] * a.drop_rs : 0.f;
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                f32x4 o = yacc[rt] * al;
#pragma unroll
                for (int r = 0; r < 4; ++r) o = mma4(zs[(16 * mt + 4 * g + r) * LS + 16 * rt + c16], p[r], o);   // Y^T[d, n] += Z^T[d, m] P[m, n]
                yacc[rt] = o;
            }
        }
        const float l = groups_sum(lsum);
        const int n = tile * 16 + c16;
        // the next tile's rows are waited for before the stores are issued (one in-order counter for loads and stores)
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        if (n < a.N) {
            // a padded token's row is 0 whatever its key row held
            const bool on = a.mask == nullptr || a.mask[(int64_t)b * a.N + n] != 0;
            const float inv = 1.f / l;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                *reinterpret_cast<f32x4*>(y + (int64_t)n * a.ys[2] + 16 * rt + 4 * g) = on ? yacc[rt] * inv : f32x4{0.f, 0.f, 0.f, 0.f};
            if (a.lse_tok && g == 0) a.lse_tok[((int64_t)b * a.H + h) * a.N + n] = (mx + __log2f(l)) * kLn2;
        }
    }
}

bool rows16(const void* p, const int64_t* s)
{
    return p == nullptr || ((reinterpret_cast<uintptr_t>(p) & 15) == 0 && s[0] % 4 == 0 && s[1] % 4 == 0 && s[2] % 4 == 0);
}

constexpr size_t kF32ScatterLdsMax = 150 * 1024;

}  // namespace

bool f32_mfma_mixer_ok(const MixerArgs& a, bool scatter)
{
    if (a.force_fma) return false;
    if (a.D != 16 && a.D != 32 && a.D != 64) return false;
    if (a.M < 16 || a.M % 16 != 0) return false;
    if (!rows16(a.q, a.qs) || !rows16(a.k, a.ks)) return false;
    if (scatter)
        return rows16(a.y, a.ys) && (reinterpret_cast<uintptr_t>(a.z) & 15) == 0 && (size_t)a.M * (a.D + 4) * 8 <= kF32ScatterLdsMax;
    return rows16(a.v, a.vs);
}

hipError_t launch_gather_f32_mfma(const MixerArgs& a, hipStream_t st)
{
    const int mblocks = (a.M + 63) / 64;
    dim3 grid(a.n_splits * mblocks, a.H, a.B);
    if (a.drop_thr != 0) {
        if (a.D == 16)      hipLaunchKernelGGL((gather_f32_mfma_kernel<16, true>), grid, dim3(256), 0, st, a);
        else if (a.D == 32) hipLaunchKernelGGL((gather_f32_mfma_kernel<32, true>), grid, dim3(256), 0, st, a);
        else                hipLaunchKernelGGL((gather_f32_mfma_kernel<64, true>), grid, dim3(256), 0, st, a);
    } else {
        if (a.D == 16)      hipLaunchKernelGGL((gather_f32_mfma_kernel<16, false>), grid, dim3(256), 0, st, a);
        else if (a.D == 32) hipLaunchKernelGGL((gather_f32_mfma_kernel<32, false>), grid, dim3(256), 0, st, a);
        else                hipLaunchKernelGGL((gather_f32_mfma_kernel<64, false>), grid, dim3(256), 0, st, a);
    }
    return hipGetLastError();
}

template <int D, bool DROP>
hipError_t scatter_launch_d(const MixerArgs& a, hipStream_t st)
{
    auto kern = scatter_f32_mfma_kernel<D, DROP>;
    const size_t lds = (size_t)a.M * (D + 4) * 8;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    // enough workgroups for four rounds of the device, each walking its share of the 64-token groups
    const int64_t groups = ((int64_t)a.N + 63) / 64;
    const int64_t want = std::max<int64_t>(1, ((int64_t)4 * device_cus() + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H));
    dim3 grid((unsigned)std::min<int64_t>(groups, want), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a);
    return hipGetLastError();
}

hipError_t launch_scatter_f32_mfma(const MixerArgs& a, hipStream_t st)
{
    if (a.drop_thr != 0) {
        if (a.D == 16) return scatter_launch_d<16, true>(a, st);
        if (a.D == 32) return scatter_launch_d<32, true>(a, st);
        return scatter_launch_d<64, true>(a, st);
    }
    if (a.D == 16) return scatter_launch_d<16, false>(a, st);
    if (a.D == 32) return scatter_launch_d<32, false>(a, st);
    return scatter_launch_d<64, false>(a, st);
}

}  // namespace flare
