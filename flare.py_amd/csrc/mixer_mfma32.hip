// FLARE mixer kernels on v_mfma_f32_32x32x16_bf16 for gfx950 (wave64): bf16, head dim 32.
//
// Operand conventions of the 32x32x16 product (c32 = lane % 32, g2 = lane / 32):
//   A (32 x 16): lane holds row c32,    k-slots 8 g2 .. 8 g2 + 7
//   B (16 x 32): lane holds column c32, k-slots 8 g2 .. 8 g2 + 7
//   D (32 x 32): lane holds column c32, register r = 4 j + i holds row 8 j + 4 g2 + i
// A contraction may visit its k index in any order as long as A and B agree, so the sixteen
// accumulators of a score tile, exponentiated and packed in pairs, ARE the two B operands of the
// value product (registers 0..7: rows 8 (e / 4) + 4 g2 + e % 4, registers 8..15: the same + 16);
// the A operand of the value product is laid out to match, once, when it is written to LDS
// (scatter) or by the addresses of the LDS transpose reads (gather).
//
// Compared with the 16x16x32 kernels this halves the number of matrix instructions per score
// (each one keeps the vector ALU from issuing for about ten cycles, which is what bounds these
// kernels), and the softmax denominators come from v_mfma_f32_4x4x4_16B_bf16 with an all-ones A
// operand, which adds the four probabilities a lane holds in two registers in one issue slot.
//
// As in the 16x16x32 kernels the steady state uses no softmax shift (fp32 and bf16 share an 8-bit
// exponent); denominators are validated afterwards and what fails is redone with a running maximum.
#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// range of an unshifted softmax denominator that proves no exponential overflowed or lost the terms that
// matter to underflow (2^-60 .. 2^120)
constexpr float kLMin = 8.6736174e-19f, kLMax = 1.329228e36f;

__device__ __forceinline__ f32x16 mma32(u32x4 a, u32x4 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// c + (sum of the four bf16 values the lane holds in p), in every register of the result
__device__ __forceinline__ f32x4 lane_sum4(u32x2 p, f32x4 c)
{
    const s16x4 ones = {0x3f80, 0x3f80, 0x3f80, 0x3f80};
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(ones, __builtin_bit_cast(s16x4, p), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float dot2_ones(uint32_t pk, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk), __builtin_bit_cast(bf16x2, 0x3f803f80u), acc, false);
}

__device__ __forceinline__ u32x4 zero4() { return u32x4{0u, 0u, 0u, 0u}; }
__device__ __forceinline__ f32x16 zero16()
{
    return f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ u32x4 load16_stream(const void* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

// multiply 8 packed bf16 by f (fp32) and repack
__device__ __forceinline__ u32x4 scale8(u32x4 v, float f)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(v[i] << 16) * f;
        const float hi = __uint_as_float(v[i] & 0xffff0000u) * f;
        o[i] = uint32_t(f32_to_bf16_bits(lo)) | (uint32_t(f32_to_bf16_bits(hi)) << 16);
    }
    return o;
}

// exponentials of the four scores of quarter Q of a tile ...
template <int Q> __device__ __forceinline__ f32x4 exp_quarter(const f32x16& s)
{
    return f32x4{fast_exp2(s[4 * Q]), fast_exp2(s[4 * Q + 1]), fast_exp2(s[4 * Q + 2]), fast_exp2(s[4 * Q + 3])};
}
// ... and their pack into the two registers they occupy in the B operands of the value product
template <int Q> __device__ __forceinline__ void pack_quarter(f32x4 e, u32x4 (&p)[2])
{
    p[Q >> 1][2 * (Q & 1)] = pack2(e[0], e[1]);
    p[Q >> 1][2 * (Q & 1) + 1] = pack2(e[2], e[3]);
}
// The order of a pipeline quarter is fixed by hand: matrix product, four exponentials (which cover its 32 cycles
// in the matrix pipe), the 4x4x4 denominator product, two packs.  The fences keep the compiler's scheduler from
// putting two matrix instructions next to each other, where the second one would stall its wave.
#define FLARE_FENCE() __builtin_amdgcn_sched_barrier(0)

// LDS transpose read: the 16 lanes of a group each name 8 bytes (4 elements) of a row-major tile; lane i of
// the group receives element i of the four 16-element rows named by lane quads 0..3.
__device__ __forceinline__ u32x2 lds_read_tr16(const void* lds_addr)
{
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    asm volatile("" ::: "memory");
    const s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)lds_addr);
    asm volatile("" ::: "memory");
    return __builtin_bit_cast(u32x2, r);
}

// c ? x : y on values (both already in registers)
__device__ __forceinline__ u32x4 pick(bool c, u32x4 x, u32x4 y) { return c ? x : y; }

__device__ __forceinline__ float max16(const f32x16& s)
{
    float m = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    return fmaxf(m, fmaxf(fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11])), fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]))));
}

// =====================================================================================
// scatter: y = softmax_m(s k q^T) z, token parallel
// =====================================================================================
// One workgroup = 4 independent waves sharing the latent operands in LDS; a wave pass covers 64 tokens (two
// column tiles of 32) against all M = 32 KS latents.  Score tile: rows = latents, columns = tokens, so that a
// token's softmax runs over the registers of its two lanes.  The unit of the software pipeline is a slot =
// (latent step, token tile): while the vector ALU exponentiates the scores of slot s, the matrix pipe computes
// the scores of slot s + 1 and the value product and the denominators of slot s - 1, issued in four quarters
// so that no matrix instruction queues behind another.  The slots of consecutive passes form one sequence: the
// last slot of a pass already computes the first scores of the next pass, whose K rows were requested one pass
// earlier.  The loop over full passes contains no branch around a memory instruction, so the compiler's wait
// for the prefetched K rows counts exactly what is outstanding instead of waiting for everything.
// A pass whose denominators leave the safe range, and a last pass that is not full, run through the exact code.
template <int KS, bool LSE>
__global__ __launch_bounds__(256, 2) void scatter32_kernel(MixerArgs a, int tokens_per_wg)
{
    constexpr int D = 32, M = 32 * KS;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem32[];
    // qa[mt][kd][lane]: A operand of the score product, latent 32 mt + c32, d = 16 kd + 8 g2 .. + 7 (log2-scaled)
    // zt[mt][hf][lane]: A operand of the value product, row c32 = output column d(c32) = 16 ((c32 >> 2) & 1) + 4 (c32 >> 3) + (c32 & 3),
    //                   k-slot e = latent 32 mt + 16 hf + 8 (e / 4) + 4 g2 + e % 4
    u32x4* qa = reinterpret_cast<u32x4*>(smem32);
    u32x4* zt = qa + KS * 128;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g2 = lane >> 5, c32 = lane & 31;
    const int h = blockIdx.y, b = blockIdx.z;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    uint16_t* y = (uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    const float* z = a.z + ((int64_t)b * a.H + h) * M * D;
    float* lse_out = LSE ? a.lse_tok + ((int64_t)b * a.H + h) * a.N : nullptr;

    for (int idx = tid; idx < KS * 128; idx += 256) {
        const int ln = idx & 63, kd = (idx >> 6) & 1, mt = idx >> 7;
        const int m = 32 * mt + (ln & 31), ch = 2 * kd + (ln >> 5);
        qa[idx] = scale8(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2);
    }
    for (int idx = tid; idx < KS * 128; idx += 256) {
        const int ln = idx & 63, hf = (idx >> 6) & 1, mt = idx >> 7;
        const int r = ln & 31, gg = ln >> 5;
        const int d = 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
        u32x4 o;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            const int e = 2 * e2;
            const int m0 = 32 * mt + 16 * hf + 8 * (e >> 2) + 4 * gg + (e & 3);
            o[e2] = uint32_t(f32_to_bf16_bits(z[(int64_t)m0 * D + d])) | (uint32_t(f32_to_bf16_bits(z[(int64_t)(m0 + 1) * D + d])) << 16);
        }
        zt[idx] = o;
    }
    __syncthreads();

    const int wg_n0 = blockIdx.x * tokens_per_wg;
    const int wg_n1 = min(a.N, wg_n0 + tokens_per_wg);
    constexpr int kStride = 4 * 64;
    const int first = wg_n0 + w * 64;
    if (first >= wg_n1) return;
    // passes of this wave that lie entirely inside the range
    const int n_full = wg_n1 - 64 - first >= 0 ? (wg_n1 - 64 - first) / kStride + 1 : 0;

    // K rows of a pass as B operands: lane (token c32 of tile tw, g2) holds d = 16 kd + 8 g2 .. + 7.  Rows past the
    // end of the range repeat its last row (tokens are columns: they never meet another token's numbers).
    auto load_k = [&](int t0, u32x4 (&dst)[2][2]) {
#pragma unroll
        for (int tw = 0; tw < 2; ++tw) {
            const int n = min(t0 + tw * 32 + c32, wg_n1 - 1);
            const uint16_t* kr = k + (int64_t)n * a.ks[2] + g2 * 8;
#pragma unroll
            for (int kd = 0; kd < 2; ++kd) dst[tw][kd] = load16_stream(kr + kd * 16);
        }
    };

    // exact code for one pass: running maximum per token, rescaling
    auto exact_pass = [&](const u32x4 (&kb)[2][2], f32x16 (&yacc)[2], float (&lrow)[2], float (&lshift)[2]) {
        asm volatile("; exact pass" ::: "memory");
        float shift[2], lsum[2];
#pragma unroll
        for (int tw = 0; tw < 2; ++tw) {
            shift[tw] = kNegBig;
            lsum[tw] = 0.f;
            yacc[tw] = zero16();
        }
#pragma unroll 1
        for (int ks = 0; ks < KS; ++ks) {
            const u32x4 q0 = qa[(2 * ks) * 64 + lane], q1 = qa[(2 * ks + 1) * 64 + lane];
            const u32x4 z0 = zt[(2 * ks) * 64 + lane], z1 = zt[(2 * ks + 1) * 64 + lane];
#pragma unroll
            for (int tw = 0; tw < 2; ++tw) {
                f32x16 s = mma32(q0, kb[tw][0], zero16());
                s = mma32(q1, kb[tw][1], s);
                const float mx = max_xor32(max16(s));
                const float nc = fmaxf(shift[tw], mx);
                const float al = fast_exp2(shift[tw] - nc);
                yacc[tw] *= al;
                lsum[tw] *= al;
                shift[tw] = nc;
                u32x4 p0, p1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    p0[e] = pack2(fast_exp2(s[2 * e] - nc), fast_exp2(s[2 * e + 1] - nc));
                    p1[e] = pack2(fast_exp2(s[8 + 2 * e] - nc), fast_exp2(s[9 + 2 * e] - nc));
                }
                float t = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    t = dot2_ones(p0[e], t);
                    t = dot2_ones(p1[e], t);
                }
                lsum[tw] += t;
                yacc[tw] = mma32(z0, p0, yacc[tw]);
                yacc[tw] = mma32(z1, p1, yacc[tw]);
            }
        }
#pragma unroll
        for (int tw = 0; tw < 2; ++tw) {
            lrow[tw] = sum_xor32(lsum[tw]);
            lshift[tw] = shift[tw];
        }
    };

    // normalise and store: lane (token c32, g2) owns d = 16 g2 .. 16 g2 + 15 (register 4 j + i: d = 16 g2 + 4 j + i)
    auto emit = [&](auto full_c, int t0, const f32x16 (&yacc)[2], const float (&lrow)[2], const float (&lshift)[2]) {
        constexpr bool FULL = decltype(full_c)::value;
        uint16_t* yr0 = y + (int64_t)(t0 + c32) * a.ys[2] + 16 * g2;
#pragma unroll
        for (int tw = 0; tw < 2; ++tw) {
            const bool in = FULL || t0 + tw * 32 + c32 < wg_n1;
            const float inv = __builtin_amdgcn_rcpf(lrow[tw]);
            uint32_t o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = pack2(yacc[tw][2 * e] * inv, yacc[tw][2 * e + 1] * inv);
            if (in) {
                uint16_t* yr = yr0 + (int64_t)tw * 32 * a.ys[2];
                __builtin_nontemporal_store(u32x4{o[0], o[1], o[2], o[3]}, reinterpret_cast<u32x4*>(yr));
                __builtin_nontemporal_store(u32x4{o[4], o[5], o[6], o[7]}, reinterpret_cast<u32x4*>(yr + 8));
            }
            // log-sum-exp of the token's scores, for the backward pass (both lanes of a token hold it; both write it,
            // which keeps the store free of a branch)
            if (LSE && in) lse_out[t0 + tw * 32 + c32] = (lshift[tw] + __log2f(lrow[tw])) * kLn2;
        }
    };

    u32x4 kb[2][2];
    int t0 = first;
    load_k(t0, kb);

    if (n_full > 0) {
        u32x4 qreg[2][2], zreg[2][2];      // by parity of the latent step
        qreg[0][0] = qa[lane];
        qreg[0][1] = qa[64 + lane];
        f32x16 sc = mma32(qreg[0][0], kb[0][0], zero16());
        sc = mma32(qreg[0][1], kb[0][1], sc);
        // every K register is consumed here once, so that no load is outstanding on the way into the loop: the
        // loop's first wait then only has to cover what an iteration itself leaves in flight
        asm volatile("" ::"v"(kb[1][0]), "v"(kb[1][1]));
#pragma unroll 1
        for (int p = 0; p < n_full; ++p, t0 += kStride) {
            u32x4 kn[2][2];
            load_k(t0 + (p + 1 < n_full ? kStride : 0), kn);     // the pass after this one (the last pass: itself, unused)
            f32x16 yacc[2];
            f32x4 dsum[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
            u32x4 pb[2] = {zero4(), zero4()};  // probabilities of the previous slot as two B operands
#pragma unroll
            for (int s = 0; s < 2 * KS; ++s) {
                const int ks = s >> 1, tw = s & 1;
                const bool last = s + 1 == 2 * KS, has_prev = s > 0;
                const int ksn = ((s + 1) >> 1) % KS, twn = (s + 1) & 1;
                const int ksp = has_prev ? (s - 1) >> 1 : 0, twp = has_prev ? (s - 1) & 1 : 0;
                if (tw == 0) {      // operands of later slots
                    zreg[ks & 1][0] = zt[(2 * ks) * 64 + lane];
                    zreg[ks & 1][1] = zt[(2 * ks + 1) * 64 + lane];
                    const int kq = (ks + 1) % KS;
                    qreg[(ks + 1) & 1][0] = qa[(2 * kq) * 64 + lane];
                    qreg[(ks + 1) & 1][1] = qa[(2 * kq + 1) * 64 + lane];
                }
                const u32x4 kn0 = last ? kn[0][0] : kb[twn][0], kn1 = last ? kn[0][1] : kb[twn][1];
                const int qpar = last ? (KS & 1) : (ksn & 1);
                f32x16 sn;
                u32x4 pc[2];
                f32x4 ex;
                // quarter 0
                sn = mma32(qreg[qpar][0], kn0, zero16());
                FLARE_FENCE();
                ex = exp_quarter<0>(sc);
                FLARE_FENCE();
                if (has_prev) dsum[twp] = lane_sum4(u32x2{pb[0][0], pb[0][1]}, dsum[twp]);
                FLARE_FENCE();
                pack_quarter<0>(ex, pc);
                FLARE_FENCE();
                // quarter 1
                if (has_prev) yacc[twp] = mma32(zreg[ksp & 1][0], pb[0], ksp == 0 ? zero16() : yacc[twp]);
                FLARE_FENCE();
                ex = exp_quarter<1>(sc);
                FLARE_FENCE();
                if (has_prev) dsum[twp] = lane_sum4(u32x2{pb[0][2], pb[0][3]}, dsum[twp]);
                FLARE_FENCE();
                pack_quarter<1>(ex, pc);
                FLARE_FENCE();
                // quarter 2
                sn = mma32(qreg[qpar][1], kn1, sn);
                FLARE_FENCE();
                ex = exp_quarter<2>(sc);
                FLARE_FENCE();
                if (has_prev) dsum[twp] = lane_sum4(u32x2{pb[1][0], pb[1][1]}, dsum[twp]);
                FLARE_FENCE();
                pack_quarter<2>(ex, pc);
                FLARE_FENCE();
                // quarter 3
                if (has_prev) yacc[twp] = mma32(zreg[ksp & 1][1], pb[1], yacc[twp]);
                FLARE_FENCE();
                ex = exp_quarter<3>(sc);
                FLARE_FENCE();
                if (has_prev) dsum[twp] = lane_sum4(u32x2{pb[1][2], pb[1][3]}, dsum[twp]);
                FLARE_FENCE();
                pack_quarter<3>(ex, pc);
                FLARE_FENCE();
                pb[0] = pc[0];
                pb[1] = pc[1];
                sc = sn;
            }
            // the last slot's value product and denominators
            {
                constexpr int ksp = KS - 1, twp = 1;
                yacc[twp] = mma32(zreg[ksp & 1][0], pb[0], ksp == 0 ? zero16() : yacc[twp]);
                dsum[twp] = lane_sum4(u32x2{pb[0][0], pb[0][1]}, dsum[twp]);
                dsum[twp] = lane_sum4(u32x2{pb[0][2], pb[0][3]}, dsum[twp]);
                yacc[twp] = mma32(zreg[ksp & 1][1], pb[1], yacc[twp]);
                dsum[twp] = lane_sum4(u32x2{pb[1][0], pb[1][1]}, dsum[twp]);
                dsum[twp] = lane_sum4(u32x2{pb[1][2], pb[1][3]}, dsum[twp]);
            }
            float lrow[2], lshift[2] = {0.f, 0.f};
            bool redo = false;
#pragma unroll
            for (int tw = 0; tw < 2; ++tw) {
                lrow[tw] = sum_xor32(dsum[tw][0]);
                redo = redo || !(lrow[tw] >= kLMin && lrow[tw] <= kLMax);
            }
            if (__builtin_expect(__any(redo), 0)) exact_pass(kb, yacc, lrow, lshift);
            emit(std::true_type{}, t0, yacc, lrow, lshift);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) kb[i][j] = kn[i][j];
        }
    }
    // what is left: at most one pass, not full
    if (t0 < wg_n1) {
        if (n_full > 0) load_k(t0, kb);
        f32x16 yacc[2];
        float lrow[2], lshift[2];
        exact_pass(kb, yacc, lrow, lshift);
        emit(std::false_type{}, t0, yacc, lrow, lshift);
    }
}

// =====================================================================================
// gather: z = softmax_n(s q k^T) v, split over N
// =====================================================================================
constexpr int kG32Tile = 128;                 // tokens per LDS tile
constexpr int kG32TileB = kG32Tile * 64;      // bytes per K or V tile (64 bytes per token row)

// One workgroup = 4 waves, 256 latents (wave w owns two latent tiles of 32), one token range.  K and V tiles of
// 128 tokens go from global memory straight into LDS (global_load_lds, 16 bytes per lane, no registers, no
// ds_write), double buffered; K chunks are XOR-swizzled on the global-address side so that the A-operand reads
// are conflict free.  Score tile: rows = tokens, columns = latents; V^T operands come from the LDS transpose
// read.  The pipeline unit is a slot = (32-token sub-tile, latent tile); sub-tiles form one sequence across
// tile boundaries, so the pipeline never drains: the single barrier per tile sits at the start of the tile's
// last sub-tile, when every read of the tile has been issued, and is followed by the loads of the tile after
// the next.
__global__ __launch_bounds__(256, 2) void gather32_kernel(MixerArgs a)
{
    constexpr int D = 32, CT = 2;
    __shared__ __attribute__((aligned(16))) uint8_t kt[2][kG32TileB];
    __shared__ __attribute__((aligned(16))) uint8_t vt[2][kG32TileB];
    __shared__ int wg_flag[4];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g2 = lane >> 5, c32 = lane & 31;
    const int mblocks = a.M / 256;
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const int m_base = mb * 256 + w * 64;

    // latent operands (B of the score product), log2-scaled
    u32x4 qb[CT][2];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int kd = 0; kd < 2; ++kd)
            qb[ct][kd] = scale8(load16(q + (int64_t)(m_base + ct * 32 + c32) * a.qs[2] + (2 * kd + g2) * 8), a.scale_log2);

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int range = max(n_end - n_begin, 0);
    const int G = (range + 31) >> 5;                   // sub-tiles of 32 tokens
    const int n_tiles = (range + kG32Tile - 1) / kG32Tile;
    const int valid_last = range - 32 * (G - 1);       // tokens of the last sub-tile (1..32)

    // tile t of the range -> LDS buffer buf.  16-byte slot p of a tile = (token p / 4, chunk position p % 4); K
    // stores chunk ch at position ch ^ ((token / 4) % 4).  Rows past the range end repeat its last row (their
    // probabilities are zeroed where they are used).
    auto stage = [&](int t, int buf) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int sb = (2 * w + j) * 64, p = sb + lane, tok = p >> 2, cp = p & 3;
            const int n = min(n_begin + t * kG32Tile + tok, n_end - 1);
            const uint16_t* kp = k + (int64_t)n * a.ks[2] + (cp ^ ((tok >> 2) & 3)) * 8;
            const uint16_t* vp = v + (int64_t)n * a.vs[2] + cp * 8;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kp,
                                             (__attribute__((address_space(3))) void*)&kt[buf][sb * 16], 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vp,
                                             (__attribute__((address_space(3))) void*)&vt[buf][sb * 16], 16, 0, 0);
        }
    };
    auto wait_stage = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

    // operands of sub-tile g: K rows (A of the score product) and V^T (A of the value product)
    auto read_k = [&](int g, u32x4 (&ka)[2]) {
        const uint8_t* base = kt[(g >> 2) & 1];
        const int tok = (g & 3) * 32 + c32;
#pragma unroll
        for (int kd = 0; kd < 2; ++kd)
            ka[kd] = *reinterpret_cast<const u32x4*>(base + tok * 64 + (((2 * kd + g2) ^ ((tok >> 2) & 3)) << 4));
    };
    auto read_v = [&](int g, u32x4 (&va)[2]) {
        const uint8_t* base = vt[(g >> 2) & 1];
        const int grp = lane >> 4, i = lane & 15;       // group: rows d = 16 (grp & 1) + i, tokens of half g2 = grp >> 1
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int t0 = (g & 3) * 32 + 16 * hf + 4 * (grp >> 1) + (i >> 2);
            const int col = (16 * (grp & 1) + 4 * (i & 3)) * 2;
            const u32x2 lo = lds_read_tr16(base + t0 * 64 + col);
            const u32x2 hi = lds_read_tr16(base + (t0 + 8) * 64 + col);
            va[hf] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    };

    float shift[CT];
    f32x16 zacc[CT];
    float lsum[CT];       // this lane's share of the denominators (its 16 tokens of every sub-tile)

    // ---- optimistic pass: no softmax shift -------------------------------------------------------------
    {
        f32x4 dsum[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            shift[ct] = 0.f;
            zacc[ct] = zero16();
            dsum[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        if (G > 0) {
            u32x4 ka[2][2], va[2][2];          // by parity of the sub-tile
            u32x4 pb[2] = {zero4(), zero4()};  // probabilities of the previous slot (none yet: zeros, met by zero values)
            va[1][0] = zero4();
            va[1][1] = zero4();
            stage(0, 0);
            wait_stage();
            __syncthreads();
            if (n_tiles > 1) stage(1, 1);
            read_k(0, ka[0]);
            read_v(0, va[0]);
            f32x16 sc = mma32(ka[0][0], qb[0][0], zero16());
            sc = mma32(ka[0][1], qb[0][1], sc);

            auto sums = [&](int ct) {
#pragma unroll
                for (int e = 0; e < 4; ++e) dsum[ct] = lane_sum4(u32x2{pb[e >> 1][2 * (e & 1)], pb[e >> 1][2 * (e & 1) + 1]}, dsum[ct]);
            };
            // One slot of the steady state: exponentials of the current scores; scores of the next slot from K operands
            // kn and latent tile CTN; value product and denominators of the previous slot (latent tile CTP) from vp.
            auto slot = [&](auto ctn_c, const u32x4 (&kn)[2], const u32x4 (&vp)[2]) {
                constexpr int CTN = decltype(ctn_c)::value, CTP = CTN;     // two latent tiles: next and previous coincide
                u32x4 pc[2];
                f32x4 ex;
                f32x16 sn = mma32(kn[0], qb[CTN][0], zero16());
                FLARE_FENCE();
                ex = exp_quarter<0>(sc);
                FLARE_FENCE();
                dsum[CTP] = lane_sum4(u32x2{pb[0][0], pb[0][1]}, dsum[CTP]);
                FLARE_FENCE();
                pack_quarter<0>(ex, pc);
                FLARE_FENCE();
                zacc[CTP] = mma32(vp[0], pb[0], zacc[CTP]);
                FLARE_FENCE();
                ex = exp_quarter<1>(sc);
                FLARE_FENCE();
                dsum[CTP] = lane_sum4(u32x2{pb[0][2], pb[0][3]}, dsum[CTP]);
                FLARE_FENCE();
                pack_quarter<1>(ex, pc);
                FLARE_FENCE();
                sn = mma32(kn[1], qb[CTN][1], sn);
                FLARE_FENCE();
                ex = exp_quarter<2>(sc);
                FLARE_FENCE();
                dsum[CTP] = lane_sum4(u32x2{pb[1][0], pb[1][1]}, dsum[CTP]);
                FLARE_FENCE();
                pack_quarter<2>(ex, pc);
                FLARE_FENCE();
                zacc[CTP] = mma32(vp[1], pb[1], zacc[CTP]);
                FLARE_FENCE();
                ex = exp_quarter<3>(sc);
                FLARE_FENCE();
                dsum[CTP] = lane_sum4(u32x2{pb[1][2], pb[1][3]}, dsum[CTP]);
                FLARE_FENCE();
                pack_quarter<3>(ex, pc);
                FLARE_FENCE();
                pb[0] = pc[0];
                pb[1] = pc[1];
                sc = sn;
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            // both slots of sub-tile g, which is not the last one (PAR = g & 1)
            auto subtile = [&](auto par_c, int g) {
                constexpr int PAR = decltype(par_c)::value;
                if (PAR == 1 && (g & 3) == 3 && (g >> 2) + 1 < n_tiles) {
                    // every read of this tile has been issued (and, by the barrier's own wait, has completed):
                    // the next tile must have landed before anyone reads it, and this tile's buffer is free
                    wait_stage();
                    __syncthreads();
                    if ((g >> 2) + 2 < n_tiles) stage((g >> 2) + 2, (g >> 2) & 1);
                }
                read_k(g + 1, ka[1 - PAR]);
                slot(I1{}, ka[PAR], va[1 - PAR]);        // slot (g, 0): next (g, 1), previous (g - 1, 1)
                read_v(g + 1, va[1 - PAR]);
                slot(I0{}, ka[1 - PAR], va[PAR]);        // slot (g, 1): next (g + 1, 0), previous (g, 0)
            };
            const int Gm = G - 1;
            int g = 0;
            for (; g + 1 < Gm; g += 2) {
                subtile(I0{}, g);
                subtile(I1{}, g + 1);
            }
            if (g < Gm) subtile(I0{}, g);

            // last sub-tile (tokens past the end of the range get probability 0), then the pipeline drains
            {
                const bool odd = (Gm & 1) != 0;
                u32x4 kl[2], vl[2], vq[2];      // K, V^T of the last sub-tile; V^T of the one before it
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    kl[i] = pick(odd, ka[1][i], ka[0][i]);
                    vl[i] = pick(odd, va[1][i], va[0][i]);
                    vq[i] = pick(odd, va[0][i], va[1][i]);
                }
                auto exps = [&](u32x4 (&pc)[2]) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int r0 = 2 * e, r1 = 2 * e + 1;
                        const bool ok0 = 8 * (r0 >> 2) + 4 * g2 + (r0 & 3) < valid_last, ok1 = 8 * (r1 >> 2) + 4 * g2 + (r1 & 3) < valid_last;
                        pc[e >> 2][e & 3] = pack2(ok0 ? fast_exp2(sc[r0]) : 0.f, ok1 ? fast_exp2(sc[r1]) : 0.f);
                    }
                };
                u32x4 pc[2];
                // slot (G - 1, 0)
                f32x16 sn = mma32(kl[0], qb[1][0], zero16());
                sn = mma32(kl[1], qb[1][1], sn);
                exps(pc);
                zacc[1] = mma32(vq[0], pb[0], zacc[1]);
                zacc[1] = mma32(vq[1], pb[1], zacc[1]);
                sums(1);
                pb[0] = pc[0]; pb[1] = pc[1]; sc = sn;
                // slot (G - 1, 1)
                exps(pc);
                zacc[0] = mma32(vl[0], pb[0], zacc[0]);
                zacc[0] = mma32(vl[1], pb[1], zacc[0]);
                sums(0);
                pb[0] = pc[0]; pb[1] = pc[1];
                // drain
                zacc[1] = mma32(vl[0], pb[0], zacc[1]);
                zacc[1] = mma32(vl[1], pb[1], zacc[1]);
                sums(1);
            }
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) lsum[ct] = dsum[ct][0];
    }

    // validate: every denominator of this wave inside the safe range, numerators finite
    bool exact;
    {
        bool bad = false;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const float l = sum_xor32(lsum[ct]);
            bad = bad || !(l <= kLMax) || (G > 0 && !(l >= kLMin));
#pragma unroll
            for (int r = 0; r < 16; ++r) bad = bad || !(fabsf(zacc[ct][r]) <= 3.0e38f);
        }
        const int anybad = __any(bad);
        __syncthreads();
        if (lane == 0) wg_flag[w] = anybad;
        __syncthreads();
        exact = (wg_flag[0] | wg_flag[1] | wg_flag[2] | wg_flag[3]) != 0;
    }
    if (exact) {
        // ---- exact pass: running maximum per latent, one tile at a time ---------------------------------
        asm volatile("; exact pass" ::: "memory");
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            shift[ct] = kNegBig;
            zacc[ct] = zero16();
            lsum[ct] = 0.f;
        }
#pragma unroll 1
        for (int t = 0; t < n_tiles; ++t) {
            __syncthreads();
            stage(t, 0);
            wait_stage();
            __syncthreads();
            const int g_end = min(G, 4 * t + 4);
#pragma unroll 1
            for (int g = 4 * t; g < g_end; ++g) {
                u32x4 ka[2], va[2];
                read_k(g & 3, ka);
                read_v(g & 3, va);
                const int valid = g == G - 1 ? valid_last : 32;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    f32x16 s = mma32(ka[0], qb[ct][0], zero16());
                    s = mma32(ka[1], qb[ct][1], s);
                    bool ok[16];
                    float mx = kNegBig;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        ok[r] = 8 * (r >> 2) + 4 * g2 + (r & 3) < valid;
                        if (ok[r]) mx = fmaxf(mx, s[r]);
                    }
                    mx = max_xor32(mx);
                    const float nc = fmaxf(shift[ct], mx);
                    const float al = fast_exp2(shift[ct] - nc);
                    zacc[ct] *= al;
                    lsum[ct] *= al;
                    shift[ct] = nc;
                    u32x4 p[2];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float p0 = ok[2 * e] ? fast_exp2(s[2 * e] - nc) : 0.f;
                        const float p1 = ok[2 * e + 1] ? fast_exp2(s[2 * e + 1] - nc) : 0.f;
                        p[e >> 2][e & 3] = pack2(p0, p1);
                    }
                    float tsum = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) tsum = dot2_ones(p[e >> 2][e & 3], tsum);
                    lsum[ct] += tsum;
                    zacc[ct] = mma32(va[0], p[0], zacc[ct]);
                    zacc[ct] = mma32(va[1], p[1], zacc[ct]);
                }
            }
        }
    }

    // partial for this split: shift (log2 units), sum, numerator, renormalised so that the sum has exponent 0
    // (keeps the merge free of overflow whatever the pass left behind)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const float l = sum_xor32(lsum[ct]);
        int e = 0;
        if (l > 0.f) (void)frexpf(l, &e);
        const float scl = l > 0.f ? ldexpf(1.f, -e) : 0.f;
        const int m = m_base + ct * 32 + c32;
        const int64_t row = (((int64_t)b * a.H + h) * a.n_parts + split) * a.M + m;
        if (g2 == 0) {
            a.part_m[row] = l > 0.f ? shift[ct] + (float)e : kNegBig;
            a.part_l[row] = l * scl;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4 o = {zacc[ct][4 * j] * scl, zacc[ct][4 * j + 1] * scl, zacc[ct][4 * j + 2] * scl, zacc[ct][4 * j + 3] * scl};
            *reinterpret_cast<f32x4*>(a.part_acc + row * D + 8 * j + 4 * g2) = o;
        }
    }
}

template <int KS, bool LSE>
hipError_t scatter32_launch_v(const MixerArgs& a, hipStream_t st)
{
    const size_t lds = (size_t)a.M * 32 * 2 * 2;
    auto kern = scatter32_kernel<KS, LSE>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    // tokens per workgroup (multiple of 256): one full round of resident workgroups when the problem is large
    // enough, so that every CU finishes at the same time
    const int slots = resident_slots(reinterpret_cast<const void*>(kern), lds);
    const int64_t per_bh = (slots + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H);
    int64_t tpw = (a.N + per_bh - 1) / per_bh;
    tpw = ((tpw + 255) / 256) * 256;
    if (tpw < 256) tpw = 256;
    dim3 grid((unsigned)((a.N + tpw - 1) / tpw), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a, (int)tpw);
    return hipGetLastError();
}

template <int KS>
hipError_t scatter32_launch(const MixerArgs& a, hipStream_t st)
{
    return a.lse_tok ? scatter32_launch_v<KS, true>(a, st) : scatter32_launch_v<KS, false>(a, st);
}

}  // namespace

// bf16, D = 32; the gather takes latent counts that are multiples of 256 and no key mask, the scatter the
// latent counts its pipeline is unrolled for.
bool mfma32_gather_supported(int dtype, int M, int D, bool masked)
{
    return dtype == 1 && D == 32 && M >= 256 && M % 256 == 0 && !masked;
}

bool mfma32_scatter_supported(int dtype, int M, int D, bool masked)
{
    return dtype == 1 && D == 32 && (M == 64 || M == 128 || M == 256 || M == 512) && !masked;
}

int mfma32_gather_resident_slots()
{
    return resident_slots(reinterpret_cast<const void*>(gather32_kernel), 0);
}

hipError_t launch_gather_mfma32(const MixerArgs& a, hipStream_t st)
{
    dim3 grid(a.n_splits * (a.M / 256), a.H, a.B);
    hipLaunchKernelGGL(gather32_kernel, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_scatter_mfma32(const MixerArgs& a, hipStream_t st)
{
    switch (a.M) {
        case 64:  return scatter32_launch<2>(a, st);
        case 128: return scatter32_launch<4>(a, st);
        case 256: return scatter32_launch<8>(a, st);
        case 512: return scatter32_launch<16>(a, st);
        default:  return hipErrorInvalidValue;
    }
}

}  // namespace flare
