// Weight and bias gradients of the fused MLP chain from the rows flare_mlp_bwd leaves:
//   dW_l[o][i] = sum_t g_out[l,t,o] a_in[l,t,i],   db_l[o] = sum_t g_out[l,t,o]        (torch: Linear's backward)
// One pass over both row arrays (bf16 / f16, C in {32, 64, 128}).  The contraction runs over tokens, so both MFMA
// operands need eight consecutive TOKENS of one channel per lane while the rows are token-major: token tiles go from
// global memory straight into LDS (16 bytes per lane, no registers) and are read back transposed
// (ds_read_b64_tr_b16).  A workgroup owns one layer and one token range and writes one partial [C,C] (+ [C]) in
// fp32; the caller sums the partials in a fixed order (no atomics).  The bias sums ride on the same A operands: one
// more product per output tile against a B operand of ones.
#include <algorithm>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mg;
template <> struct Mg<bf16_t> {
    static constexpr uint32_t kOnes = 0x3F803F80u;
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mg<f16_t> {
    static constexpr uint32_t kOnes = 0x3C003C00u;
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

// Transposed 64-bit LDS read: the 16 lanes of a group read a block of 4 rows x 16 columns of 16-bit elements
// (lane j points at row j / 4, columns 4 (j % 4) .. + 3) and lane j receives column j of the four rows.
// Issued as an asm statement: the compiler orders every LDS read it knows of behind ALL loads-into-LDS in flight
// (it cannot tell the ring slots apart), which would undo the prefetch of the later tiles.  The result is valid
// only after lds_wait() below.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x2 read_tr16(uint32_t lds_byte_addr)
{
    u32x2 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r) : "v"(lds_byte_addr) : "memory");
    return r;
}
// all LDS reads of this wave have returned; the operands pass through the statement so that nothing uses them earlier
template <int N>
__device__ __forceinline__ void lds_wait(u32x2 (&r)[N])
{
    static_assert(N == 8 || N == 12, "operand halves of one k-step");
    if constexpr (N == 8)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]) :: "memory");
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]),
                     "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]) :: "memory");
}

constexpr int kStages = 3;      // ring of token tiles in LDS; two tiles are in flight while one is read

// Waves of a workgroup: WO x WI tile the [C/16] x [C/16] grid of 16 x 16 output blocks, WK split the tokens of a tile.
template <typename T, int C, int WO, int WI, int WK>
__global__ __launch_bounds__(64 * WO * WI * WK) void mlp_wgrad_kernel(MlpWgradArgs a)
{
    constexpr int NW = WO * WI * WK, NT = 64 * NW;
    constexpr int FT = C / 16, OT = FT / WO, IT = FT / WI;
    constexpr int KT = 32 * WK;                 // tokens per tile
    constexpr int CPR = C / 8;                  // 16-byte chunks per row
    constexpr int ROWB = C * 2;
    constexpr int TILEB = KT * ROWB;            // one operand's tile
    constexpr int NCH = 2 * KT * CPR / NT;      // chunks per thread and tile (both operands)
    static_assert((2 * KT * CPR) % NT == 0 && (KT * CPR) % 64 == 0, "a wave's 64 chunks lie in one operand");
    using M_ = Mg<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];      // [kStages][2 operands][KT][ROWB]

    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;       // the low half of a generic LDS address is the LDS byte address

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = w / (WO * WI), wo = (w / WI) % WO, wi = w % WI;
    const int l = blockIdx.y;
    const int64_t t0 = (int64_t)blockIdx.x * a.tokens_per_wg;
    const int64_t t1 = t0 + a.tokens_per_wg < a.T ? t0 + a.tokens_per_wg : a.T;
    const int ns = (int)((t1 - t0 + KT - 1) / KT);
    const uint16_t* gl = a.g_out + (size_t)l * a.g_lstride;
    const uint16_t* al = a.a_in + (size_t)l * a.a_lstride;

    // 16-byte chunk c of a row of token `tok` (tile-relative) sits at chunk c ^ swz(tok): the transposed reads of a
    // wave touch 16 consecutive rows, which without the key would all start in the same bank
    auto swz = [](int tok) { return 2 * (tok & (C / 16 - 1)); };

    // tile s of the range -> ring slot s % kStages.  Rows past the end of the array are read from its last row (the
    // products mask them out); tiles past the range are requested all the same so that the count of loads in flight
    // is the same in every iteration.
    auto request = [&](int s) {
        uint8_t* slot = smem + (s % kStages) * 2 * TILEB;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c0 = i * NT + w * 64;                          // uniform over the wave
            const int op = c0 / (KT * CPR);                          // 0: g_out, 1: a_in
            const int rem = (c0 - op * KT * CPR) + lane;
            const int tok = rem / CPR, chl = rem % CPR;
            int64_t t = t0 + (int64_t)s * KT + tok;
            t = t < a.T ? t : a.T - 1;
            const uint16_t* src = (op ? al : gl) + (size_t)t * C + ((chl ^ swz(tok)) << 3);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(slot + c0 * 16), 16, 0, 0);
        }
    };

    f32x4 acc[OT][IT], accb[OT];
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) {
        accb[ot] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int it = 0; it < IT; ++it) acc[ot][it] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const u32x4 ones = {M_::kOnes, M_::kOnes, M_::kOnes, M_::kOnes};

#pragma unroll
    for (int s = 0; s < kStages - 1; ++s) request(s);

    for (int s = 0; s < ns; ++s) {
        // this thread's loads of tile s have landed (results return in order: the kStages - 2 later tiles may stay
        // in flight), then everybody's have, and nobody reads tile s - 1 any more: its slot takes tile s + kStages - 1
        if constexpr (kStages == 3) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NCH) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // the bare barrier instruction: __syncthreads() would add a fence that waits for every load in flight, the
        // later tiles included.  Nothing else needs ordering here: the tiles are written by the loads just waited for
        // and read by LDS instructions whose results the products below have already consumed.
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        request(s + kStages - 1);

        const int64_t tb = t0 + (int64_t)s * KT + wk * 32;            // first token of this wave's k-step
        if (tb >= t1) continue;
        const uint32_t gt = lds0 + (s % kStages) * 2 * TILEB, at = gt + TILEB;
        // lane (g, c16) of a transposed read: row 4 g + c16 / 4 (and 16 further), 8-byte piece c16 % 4 of the tile's 32 bytes
        const int r0 = wk * 32 + 4 * g + (c16 >> 2), r1 = r0 + 16;
        const int piece = ((c16 & 3) >> 1), sub = (c16 & 1) << 3;
        u32x2 half[2 * (OT + IT)];
#pragma unroll
        for (int i = 0; i < OT + IT; ++i) {
            const int ft = i < OT ? wo * OT + i : wi * IT + (i - OT);
            const uint32_t tile = i < OT ? gt : at;
            const int ch = 2 * ft + piece;
            half[2 * i] = read_tr16(tile + r0 * ROWB + ((ch ^ swz(r0)) << 4) + sub);
            half[2 * i + 1] = read_tr16(tile + r1 * ROWB + ((ch ^ swz(r1)) << 4) + sub);
        }
        lds_wait(half);
        u32x4 A[OT], B[IT];
#pragma unroll
        for (int ot = 0; ot < OT; ++ot) A[ot] = u32x4{half[2 * ot][0], half[2 * ot][1], half[2 * ot + 1][0], half[2 * ot + 1][1]};
#pragma unroll
        for (int it = 0; it < IT; ++it)
            B[it] = u32x4{half[2 * (OT + it)][0], half[2 * (OT + it)][1], half[2 * (OT + it) + 1][0], half[2 * (OT + it) + 1][1]};
        if (tb + 32 > t1) {
            // the range ends inside this k-step: k-slot j of the operand is token 4 g + j (j < 4) or 16 + 4 g + j - 4
            const int left = (int)(t1 - tb);
#pragma unroll
            for (int ot = 0; ot < OT; ++ot)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int tok = (j < 4 ? 0 : 12) + 4 * g + j;
                    if (tok >= left) A[ot][j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
                }
        }
#pragma unroll
        for (int ot = 0; ot < OT; ++ot) {
#pragma unroll
            for (int it = 0; it < IT; ++it) acc[ot][it] = M_::mma(A[ot], B[it], acc[ot][it]);
            if (wi == 0) accb[ot] = M_::mma(A[ot], ones, accb[ot]);
        }
    }
    // drain the requests that ran past the range before the workgroup ends
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // accumulator of a 16 x 16 block: lane (g, c16) holds rows 4 g .. 4 g + 3 (output channels) of column c16 (input channel)
    const size_t part = ((size_t)blockIdx.x * WK + wk) * a.L + l;
    float* dw = a.dw_part + part * C * C;
#pragma unroll
    for (int ot = 0; ot < OT; ++ot)
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                dw[(size_t)(16 * (wo * OT + ot) + 4 * g + r) * C + 16 * (wi * IT + it) + c16] = acc[ot][it][r];
    if (wi == 0 && c16 == 0 && a.db_part) {
        float* db = a.db_part + part * C;
#pragma unroll
        for (int ot = 0; ot < OT; ++ot)
            *reinterpret_cast<f32x4*>(db + 16 * (wo * OT + ot) + 4 * g) = accb[ot];
    }
}

// out[i] = sum over p of part[p][i].  Thread (x, y) of a 64 x 4 workgroup: four outputs, the partials p = y, y + 4,
// ... with four loads in flight; the four y meet in LDS.  The order of the additions is fixed.
__global__ __launch_bounds__(256) void sum_parts_kernel(const float* part, int parts, int64_t n, float* out)
{
    __shared__ f32x4 red[4][64];
    const int x = threadIdx.x & 63, y = threadIdx.x >> 6;
    const int64_t i = ((int64_t)blockIdx.x * 64 + x) * 4;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < n) {
        int p = y;
        for (; p + 12 < parts; p += 16) {
            const f32x4 v0 = *reinterpret_cast<const f32x4*>(part + (size_t)p * n + i);
            const f32x4 v1 = *reinterpret_cast<const f32x4*>(part + (size_t)(p + 4) * n + i);
            const f32x4 v2 = *reinterpret_cast<const f32x4*>(part + (size_t)(p + 8) * n + i);
            const f32x4 v3 = *reinterpret_cast<const f32x4*>(part + (size_t)(p + 12) * n + i);
            s += (v0 + v1) + (v2 + v3);
        }
        for (; p < parts; p += 4) s += *reinterpret_cast<const f32x4*>(part + (size_t)p * n + i);
    }
    red[y][x] = s;
    __syncthreads();
    if (y == 0 && i < n) *reinterpret_cast<f32x4*>(out + i) = (red[0][x] + red[1][x]) + (red[2][x] + red[3][x]);
}

template <int C> struct WgradShape;
template <> struct WgradShape<128> { static constexpr int WO = 4, WI = 2, WK = 1; };
template <> struct WgradShape<64>  { static constexpr int WO = 2, WI = 2, WK = 2; };
template <> struct WgradShape<32>  { static constexpr int WO = 1, WI = 1, WK = 8; };

template <typename T, int C>
hipError_t launch_c(const MlpWgradArgs& a, hipStream_t st)
{
    using S = WgradShape<C>;
    auto kern = mlp_wgrad_kernel<T, C, S::WO, S::WI, S::WK>;
    const size_t lds = (size_t)kStages * 2 * (32 * S::WK) * C * 2;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    const int64_t n_wg = (a.T + a.tokens_per_wg - 1) / a.tokens_per_wg;
    hipLaunchKernelGGL(kern, dim3((unsigned)n_wg, (unsigned)a.L), dim3(64 * S::WO * S::WI * S::WK), lds, st, a);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_t(const MlpWgradArgs& a, hipStream_t st)
{
    switch (a.C) {
        case 32:  return launch_c<T, 32>(a, st);
        case 64:  return launch_c<T, 64>(a, st);
        case 128: return launch_c<T, 128>(a, st);
        default:  return hipErrorInvalidValue;
    }
}

int wgrad_wk(int C) { return C == 128 ? 1 : C == 64 ? 2 : 8; }

}  // namespace

// Tokens per workgroup: at least one workgroup per compute unit over all layers, between 1024 and 4096 tokens (more,
// smaller ranges only add partial results to write and sum: measured at 262,144 tokens x 5 layers), a multiple of the
// kernel's token tile.
int64_t mlp_wgrad_tokens_per_wg(int64_t T, int C, int L)
{
    const int64_t kt = 32 * wgrad_wk(C);
    int64_t want = (T * L + (int64_t)device_cus() - 1) / (int64_t)device_cus();
    want = std::min<int64_t>(std::max<int64_t>(want, 1024), 4096);
    return (want + kt - 1) / kt * kt;
}

// partial results a launch writes (token ranges x the kernel's split of a token tile over waves)
int mlp_wgrad_partials(int64_t T, int C, int L)
{
    const int64_t per = mlp_wgrad_tokens_per_wg(T, C, L);
    return (int)((T + per - 1) / per) * wgrad_wk(C);
}

hipError_t launch_mlp_wgrad(const MlpWgradArgs& a0, int w_dtype, hipStream_t st)
{
    MlpWgradArgs a = a0;
    a.tokens_per_wg = mlp_wgrad_tokens_per_wg(a.T, a.C, a.L);
    hipError_t e = w_dtype == 1 ? launch_t<bf16_t>(a, st) : launch_t<f16_t>(a, st);
    if (e != hipSuccess) return e;
    const int parts = mlp_wgrad_partials(a.T, a.C, a.L);
    if (a.dw) {
        const int64_t n = (int64_t)a.L * a.C * a.C;
        hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((n / 4 + 63) / 64)), dim3(256), 0, st, a.dw_part, parts, n, a.dw);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (a.db && a.db_part) {
        const int64_t n = (int64_t)a.L * a.C;
        hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((n / 4 + 63) / 64)), dim3(256), 0, st, a.db_part, parts, n, a.db);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace flare
