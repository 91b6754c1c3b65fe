// Backward of the FLARE mixer on v_mfma_f32_32x32x16_bf16 (bf16, head dim 32): the dz pass, the token pass and the dq pass.
//
//   dz_m = sum_n Bt[n,m] dy_n,  Bt[n,m] = exp2(S[n,m] - rho2_n) <= 1   (S in log2 units, rho2_n = the token's
//   log-sum-exp over the latents, saved by the forward's scatter),  and beside it  delta_n = <dy_n, y_n>.
//
// This is the forward gather with dY in the place of V and a per-token shift instead of a softmax over tokens, so it has
// the gather's shape (mixer_mfma32.hip): one workgroup = 4 waves that own the same 32 MT latents and different tokens,
// wave w takes the 32-token passes w, w + 4, ... of the workgroup's token range; K rows go straight from global memory
// into A operands, the latent operands sit in LDS in operand order, dY^T comes from a wave-private LDS tile through
// the transposing read; no barrier in the token loop; the matrix pipe computes the scores of slot s + 1 and the value
// product of slot s - 1 while the vector ALU exponentiates slot s.  The shift costs no instruction: -rho2_n is a row
// vector of the score tile (rows = tokens), i.e. the initial accumulator of its first matrix product.  The lane's
// sixteen rows reach it through a wave-private LDS row of 32 floats, one pass ahead.
// Every weight is <= 1: no validation, no exact path.  The four waves' sums meet in LDS in a fixed order and the
// workgroup writes one partial (summed over the splits by bwd_merge_kernel<0> of mixer_bwd_mfma.hip).
#include <type_traits>

#include "common.hpp"
#include "mfma32.hpp"

namespace flare {

namespace {

// (the words go through scalar copies: a bit cast applied to a vector element directly was compiled as a cast of word 0)
__device__ __forceinline__ float dot2_bf16(uint32_t x, uint32_t y, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, y), acc, false);
}
__device__ __forceinline__ float dot8_bf16(u32x4 x, u32x4 y)
{
    return dot2_bf16(x[3], y[3], dot2_bf16(x[2], y[2], dot2_bf16(x[1], y[1], dot2_bf16(x[0], y[0], 0.f))));
}

template <int MT>
__global__ __launch_bounds__(256, 2) void bwd_dz32_kernel(MixerBwdArgs a)
{
    constexpr int D = 32;
    static_assert(MT >= 2, "at least two latent tiles per wave");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem32z[];
    u32x4* qb = reinterpret_cast<u32x4*>(smem32z);              // [MT][2][64]: B operands of the score product

    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g2 = lane >> 5, c32 = lane & 31;
    uint8_t* vb = smem32z + MT * 2048 + w * 2048;               // this wave's dY tile: 32 rows of 64 bytes
    float* rb = reinterpret_cast<float*>(smem32z + MT * 2048 + 4 * 2048) + w * 32;      // this wave's row of -rho2
    float* wmax = reinterpret_cast<float*>(smem32z + MT * 2048 + 4 * 2048 + 4 * 128);   // [4]
    const int mblocks = a.M / (32 * MT);
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* dy = (const uint16_t*)a.dy + b * a.dys[0] + h * a.dys[1];
    const uint16_t* yv = (const uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    const float* rho = a.lse_tok + bh * a.N;
    float* dlt = a.delta_tok + bh * a.N;
    const int m_base = mb * 32 * MT;
    // the first latent block also produces delta_n = <dy_n, y_n> and the smallest rho2_n of the split for the later passes
    const bool make_delta = mb == 0;

    for (int idx = tid; idx < MT * 128; idx += 256) {
        const int ln = idx & 63, kd = (idx >> 6) & 1, mt = idx >> 7;
        const int m = m_base + 32 * mt + (ln & 31), ch = 2 * kd + (ln >> 5);
        qb[idx] = scale8(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2);
    }
    __syncthreads();

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int n_last = max(n_end - 1, 0);
    const int first = n_begin + 32 * w;
    const int n_full = first + 32 <= n_end ? (n_end - 32 - first) / 128 + 1 : 0;   // passes of this wave inside the range
    const int tail0 = first + 128 * n_full;                                          // start of a last, shorter pass
    const int tail_valid = tail0 < n_end ? n_end - tail0 : 0;                        // its tokens (0: none)

    // K rows of a pass as A operands: lane (token c32, g2) holds d = 16 kd + 8 g2 .. + 7.  dY (and Y) rows as they are
    // written to the LDS tile: lane l holds the 16-byte chunk l % 4 of row 16 j + l / 4.  Rows past the end of the
    // range repeat its last row (their weights are zero: their shift is set to -3e38 where it is staged).
    auto load_k = [&](int n0, u32x4 (&dst)[2]) {
        const uint16_t* kr = k + (int64_t)min(n0 + c32, n_last) * a.ks[2] + g2 * 8;
        dst[0] = load16_stream(kr);
        dst[1] = load16_stream(kr + 16);
    };
    auto load_rows = [&](const uint16_t* base, int64_t stride, int n0, u32x4 (&dst)[2]) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            dst[j] = load16_stream(base + (int64_t)min(n0 + 16 * j + (lane >> 2), n_last) * stride + (lane & 3) * 8);
    };
    auto load_r = [&](int n0) { return rho[min(n0 + c32, n_last)]; };
    auto put_v = [&](const u32x4 (&src)[2]) {
#pragma unroll
        for (int j = 0; j < 2; ++j) *reinterpret_cast<u32x4*>(vb + (j * 64 + lane) * 16) = src[j];
    };
    // A operands of the value product: row d = c32, k-slot e of half hf = token 16 hf + 8 (e / 4) + 4 g2 + e % 4
    auto read_v = [&](u32x4 (&va)[2]) {
        const int grp = lane >> 4, i = lane & 15;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int t0 = 16 * hf + 4 * (grp >> 1) + (i >> 2);
            const int col = (16 * (grp & 1) + 4 * (i & 3)) * 2;
            const u32x2 lo = lds_read_tr16(vb + t0 * 64 + col);
            const u32x2 hi = lds_read_tr16(vb + (t0 + 8) * 64 + col);
            va[hf] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    };
    // The lanes hand each other their tokens' shifts through the wave's LDS row.  To the compiler every lane is a thread
    // of its own: the fences keep a lane's reads of other lanes' entries behind its own store.
    float rmax = -3.0e38f;      // largest -rho2 among the tokens this lane staged (inside the range)
    auto put_r = [&](float r, int n0) {
        const bool in = n0 + c32 < n_end;
        const float nr = in ? -r * kLog2e : -3.0e38f;
        if (in) rmax = fmaxf(rmax, nr);
        asm volatile("" ::: "memory");
        if (g2 == 0) rb[c32] = nr;
        asm volatile("" ::: "memory");
    };
    auto read_r = [&]() {
        f32x16 o;
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(rb + 8 * j + 4 * g2);
            o[4 * j] = t[0]; o[4 * j + 1] = t[1]; o[4 * j + 2] = t[2]; o[4 * j + 3] = t[3];
        }
        asm volatile("" ::: "memory");
        return o;
    };
    // delta_n = <dy_n, y_n> of the 32 tokens of a pass: four lanes per token
    auto put_delta = [&](const u32x4 (&dyr)[2], const u32x4 (&yr)[2], int n0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            float pd = dot8_bf16(dyr[j], yr[j]);
            pd += __shfl_xor(pd, 1);
            pd += __shfl_xor(pd, 2);
            const int n = n0 + 16 * j + (lane >> 2);
            if ((lane & 3) == 0 && n < n_end) dlt[n] = pd;
        }
    };

    f32x16 zacc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) zacc[mt] = zero16();

    if (n_full > 0) {
        u32x4 kb[2], kn[2], vr[2], yr[2] = {zero4(), zero4()};
        u32x4 va[2] = {zero4(), zero4()};
        u32x4 pb[2] = {zero4(), zero4()};      // weights of the previous slot (none yet: zeros, met by zero values)
        u32x4 qreg[2];
        load_k(first, kb);
        load_rows(dy, a.dys[2], first, vr);
        if (make_delta) load_rows(yv, a.ys[2], first, yr);
        put_r(load_r(first), first);
        f32x16 nr = read_r();
        float rn = load_r(first + 128);
        qreg[0] = qb[lane];
        qreg[1] = qb[64 + lane];
        f32x16 sc = mma32(kb[0], qreg[0], nr);
        sc = mma32(kb[1], qreg[1], sc);
        qreg[0] = qb[2 * 64 + lane];
        qreg[1] = qb[3 * 64 + lane];

        // One slot: exponentials of the current scores (sc); scores of the next slot (latent tile (S + 1) % MT, of the
        // next pass's rows in the last slot); value product of the previous slot.  The shifts of the next pass (staged
        // in the wave's LDS row at the start of this pass) replace this pass's once its last score tile has started.
        auto slot = [&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            constexpr bool LAST = S + 1 == MT;
            constexpr int PREV = (S + MT - 1) % MT;
            constexpr int QF = (S + 2) % MT;
            const u32x4 kx0 = LAST ? kn[0] : kb[0], kx1 = LAST ? kn[1] : kb[1];
            f32x16 sn;
            u32x4 pc[2];
            f32x4 ex;
            // quarter 0
            sn = mma32(kx0, qreg[0], nr);
            FLARE_FENCE();
            if constexpr (S + 2 == MT) nr = read_r();
            qreg[0] = qb[(2 * QF) * 64 + lane];
            ex = exp_quarter<0>(sc);
            FLARE_FENCE();
            pack_quarter<0>(ex, pc);
            FLARE_FENCE();
            // quarter 1
            zacc[PREV] = mma32(va[0], pb[0], zacc[PREV]);
            FLARE_FENCE();
            ex = exp_quarter<1>(sc);
            FLARE_FENCE();
            pack_quarter<1>(ex, pc);
            FLARE_FENCE();
            // quarter 2
            sn = mma32(kx1, qreg[1], sn);
            FLARE_FENCE();
            qreg[1] = qb[(2 * QF + 1) * 64 + lane];
            ex = exp_quarter<2>(sc);
            FLARE_FENCE();
            pack_quarter<2>(ex, pc);
            FLARE_FENCE();
            // quarter 3
            zacc[PREV] = mma32(va[1], pb[1], zacc[PREV]);
            FLARE_FENCE();
            if constexpr (S == 0) read_v(va);      // this pass's dY^T, after the last product with the previous pass's
            ex = exp_quarter<3>(sc);
            FLARE_FENCE();
            pack_quarter<3>(ex, pc);
            FLARE_FENCE();
            pb[0] = pc[0];
            pb[1] = pc[1];
            sc = sn;
        };

        int n0 = first;
#pragma unroll 1
        for (int p = 0; p < n_full; ++p, n0 += 128) {
            put_v(vr);
            if (make_delta) put_delta(vr, yr, n0);
            put_r(rn, n0 + 128);           // the next pass's shifts (rows past the range: no weight)
            // the next pass's rows; the last pass requests rows of the range again (unused)
            load_k(n0 + 128, kn);
            load_rows(dy, a.dys[2], n0 + 128, vr);
            if (make_delta) load_rows(yv, a.ys[2], n0 + 128, yr);
            rn = load_r(n0 + 256);
            static_for<0, MT>(slot);
            kb[0] = kn[0];
            kb[1] = kn[1];
        }
        // drain: the last slot's value product
        zacc[MT - 1] = mma32(va[0], pb[0], zacc[MT - 1]);
        zacc[MT - 1] = mma32(va[1], pb[1], zacc[MT - 1]);
    }

    // the shorter last pass of a range, without pipelining
    if (tail_valid > 0) {
        u32x4 kb[2], vr[2], yr[2], va[2];
        load_k(tail0, kb);
        load_rows(dy, a.dys[2], tail0, vr);
        if (make_delta) {
            load_rows(yv, a.ys[2], tail0, yr);
            put_delta(vr, yr, tail0);
        }
        put_v(vr);
        read_v(va);
        put_r(load_r(tail0), tail0);
        const f32x16 nr = read_r();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const u32x4 q0 = qb[(2 * mt) * 64 + lane], q1 = qb[(2 * mt + 1) * 64 + lane];
            f32x16 s = mma32(kb[0], q0, nr);
            s = mma32(kb[1], q1, s);
            u32x4 p[2];
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e >> 2][e & 3] = pack2(fast_exp2(s[2 * e]), fast_exp2(s[2 * e + 1]));
            zacc[mt] = mma32(va[0], p[0], zacc[mt]);
            zacc[mt] = mma32(va[1], p[1], zacc[mt]);
        }
    }

    // ---- the four waves' sums meet in LDS: (w0 + w2) + (w1 + w3) --------------------------------------------
    constexpr int kSlotB = MT * 4 * 64 * 16;
    auto publish = [&](int slot_i) {
        f32x4* z4 = reinterpret_cast<f32x4*>(smem32z + slot_i * kSlotB);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                z4[(mt * 4 + j) * 64 + lane] = f32x4{zacc[mt][4 * j], zacc[mt][4 * j + 1], zacc[mt][4 * j + 2], zacc[mt][4 * j + 3]};
    };
    auto absorb = [&](int slot_i) {
        const f32x4* z4 = reinterpret_cast<const f32x4*>(smem32z + slot_i * kSlotB);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 o = z4[(mt * 4 + j) * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; ++i) zacc[mt][4 * j + i] += o[i];
            }
    };
    // the smallest rho2 of the split (= minus the largest -rho2 any wave staged), before the LDS is reused
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) rmax = fmaxf(rmax, __shfl_xor(rmax, o));
    __syncthreads();
    if (lane == 0) wmax[w] = rmax;
    __syncthreads();
    if (make_delta && tid == 0)
        a.rho_min[bh * a.n_splits + split] = -fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    __syncthreads();
    if (w >= 2) publish(w - 2);
    __syncthreads();
    if (w < 2) absorb(w);
    __syncthreads();
    if (w == 1) publish(0);
    __syncthreads();
    if (w == 0) {
        absorb(0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m_base + mt * 32 + c32;
            const int64_t row = (bh * a.n_splits + split) * a.M + m;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<f32x4*>(a.part + row * D + 8 * j + 4 * g2) =
                    f32x4{zacc[mt][4 * j], zacc[mt][4 * j + 1], zacc[mt][4 * j + 2], zacc[mt][4 * j + 3]};
        }
    }
}

// =====================================================================================
// dq pass: dq_m = s sum_n dS[m,n] k_n
// =====================================================================================
// Same shape again (one workgroup = 4 waves x the same 32 MT latents x different 32-token passes; no barrier in the token
// loop).  Per (pass, latent tile) the score-like tiles have rows = tokens and the lane's column = one latent:
//   S = K q^T (log2 units),   g = V dz^T + (eR dY)(eL z)^T   in ONE accumulator chain,
//   dS' = exp2(S) (g - eL_m (eR delta)_n - Delta_m),          dq'^T += K^T dS'   (K^T from the wave's LDS tile of K rows)
// (the two per-latent terms are one more matrix product on g's chain: two vector instructions per score, exp and multiply)
// and dq_m = s c_m dq'_m with c_m = exp2(-L2_m) applied once, where the partial is written.  This is the
// one-exponential form of mixer_bwd_mfma.hip (Bt = A eL[m] eR[n], eL[m] = exp2(L2_m - Lmax2), eR[n] = exp2(Lmax2 - rho2_n))
// with the gather's weight A = exp2(S - L2_m) split into exp2(S) and the per-latent constant c_m, which is exact while
// every |L2_m| of the (b,h) stays below 60 (bwd_unshifted_form: checked per (b,h), together with the condition of the
// one-exponential form itself).  eR meets the dY rows where a lane holds them as its own token's A operand (a per-lane
// factor); eL meets the z operands when they are staged.  A (b,h) outside these conditions takes the general form with
// both exponentials and every term element by element, in the plain (unpipelined) pass that also serves ragged ends.

// x rounded to bf16, as a float
__device__ __forceinline__ float bf16_head(float x) { return __uint_as_float(pack2(x, 0.f) << 16); }

// 8 packed bf16 times f, repacked by the conversion instruction
__device__ __forceinline__ u32x4 scale8_cvt(u32x4 v, float f)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = v[i];
        o[i] = pack2(__uint_as_float(w << 16) * f, __uint_as_float(w & 0xffff0000u) * f);
    }
    return o;
}

__device__ __forceinline__ u32x4 pack8f(const float* p, float f)
{
    const f32x4 a = *reinterpret_cast<const f32x4*>(p) * f, b = *reinterpret_cast<const f32x4*>(p + 4) * f;
    return u32x4{pack2(a[0], a[1]), pack2(a[2], a[3]), pack2(b[0], b[1]), pack2(b[2], b[3])};
}

template <int MT>
__global__ __launch_bounds__(256, 2) void bwd_dq32_kernel(MixerBwdArgs a)
{
    constexpr int D = 32;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem32q[];
    u32x4* qb = reinterpret_cast<u32x4*>(smem32q);              // [MT][2][64]: q (log2-scaled), B operands
    u32x4* dzb = qb + MT * 128;                                 // dz
    u32x4* zb = dzb + MT * 128;                                 // z (times eL in the one-exponential form)
    u32x4* xb = zb + MT * 128;                                  // [MT][64]: per-latent scalars as one more B operand (below)

    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g2 = lane >> 5, c32 = lane & 31;
    uint8_t* kt = smem32q + 3 * MT * 2048 + MT * 1024 + w * 2048;           // this wave's K tile: 32 rows of 64 bytes
    float* rb = reinterpret_cast<float*>(smem32q + 3 * MT * 2048 + MT * 1024 + 4 * 2048) + w * 64;   // two rows of 32 per-token scalars
    // Workgroups are dealt to the eight XCDs in turn (each with an L2 of its own): the latent blocks of one token range sit
    // eight workgroup numbers apart, so they run on the same XCD at about the same time and the K, V and dY rows of the
    // range come from HBM once.
    const int mblocks = a.M / (32 * MT);
    const int grp = blockIdx.x / (8 * mblocks), rem = blockIdx.x % (8 * mblocks);
    const int split = grp * 8 + (rem & 7), mb = rem >> 3;
    if (split >= a.n_splits) return;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint16_t* dy = (const uint16_t*)a.dy + b * a.dys[0] + h * a.dys[1];
    const float* rho = a.lse_tok + bh * a.N;
    const float* dlt = a.delta_tok + bh * a.N;
    const int m_base = mb * 32 * MT;

    // Which form the (b,h) takes: every wave computes the same answer.
    float lmax2;
    const bool fast = bwd_unshifted_form(a, bh, lane, lmax2);

    // per-latent scalars of the lane's column in every tile
    float l2m[MT], dm[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m_base + 32 * mt + c32;
        l2m[mt] = a.lse_lat[bh * a.M + m] * kLog2e;
        dm[mt] = a.delta_lat[bh * a.M + m];
    }
    for (int idx = tid; idx < MT * 128; idx += 256) {
        const int ln = idx & 63, kd = (idx >> 6) & 1, mt = idx >> 7;
        const int m = m_base + 32 * mt + (ln & 31), ch = 2 * kd + (ln >> 5);
        qb[idx] = scale8(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2);
        dzb[idx] = pack8f(a.dz + (bh * a.M + m) * D + ch * 8, 1.f);
        zb[idx] = pack8f(a.z + (bh * a.M + m) * D + ch * 8, fast ? fast_exp2(a.lse_lat[bh * a.M + m] * kLog2e - lmax2) : 1.f);
    }
    // The two per-latent terms of the one-exponential form, -eL_m (eR delta)_n - Delta_m, are a contraction over two more
    // "features" and ride on one more matrix product instead of two vector instructions per score: B operand
    // (-eL, -Delta) of the latent against A operand ((eR delta)_n, 1) of the token.  Both sides are split into a bf16
    // head and tail (the cross term of the two tails is dropped: 2^-16 relative), so the terms keep 16 bits.
    for (int idx = tid; idx < MT * 64; idx += 256) {
        const int ln = idx & 63, mt = idx >> 6;
        const int m = m_base + 32 * mt + (ln & 31);
        const float el = fast_exp2(a.lse_lat[bh * a.M + m] * kLog2e - lmax2), de = a.delta_lat[bh * a.M + m];
        const float el_h = bf16_head(el), de_h = bf16_head(de);
        const u32x4 o = {pack2(-el_h, -el_h), pack2(-(el - el_h), -de_h), pack2(-(de - de_h), 0.f), 0u};
        xb[idx] = (ln >> 5) == 0 ? o : zero4();
    }
    __syncthreads();

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int n_last = max(n_end - 1, 0);
    const int first = n_begin + 32 * w;
    const int n_full = first + 32 <= n_end ? (n_end - 32 - first) / 128 + 1 : 0;
    const int tail0 = first + 128 * n_full;
    const int tail_valid = tail0 < n_end ? n_end - tail0 : 0;

    // rows of a pass as A operands: lane (token c32, g2) holds d = 16 kd + 8 g2 .. + 7 of its token
    auto load_a = [&](const uint16_t* base, int64_t stride, int n0, u32x4 (&dst)[2]) {
        // (plain loads: the workgroup of the other latent block reads the same rows from the L2 a moment later)
        const uint16_t* r = base + (int64_t)min(n0 + c32, n_last) * stride + g2 * 8;
        dst[0] = load16(r);
        dst[1] = load16(r + 16);
    };
    // the K rows a lane holds as A operands, written to the wave's tile (row c32, 16-byte chunk 2 kd + g2) ...
    auto put_k = [&](const u32x4 (&src)[2]) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int kd = 0; kd < 2; ++kd) *reinterpret_cast<u32x4*>(kt + c32 * 64 + (2 * kd + g2) * 16) = src[kd];
        asm volatile("" ::: "memory");
    };
    // ... and taken back transposed: row d = c32, k-slot e of half hf = token 16 hf + 8 (e / 4) + 4 g2 + e % 4
    auto read_kt = [&](u32x4 (&ka)[2]) {
        const int grp = lane >> 4, i = lane & 15;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int t0 = 16 * hf + 4 * (grp >> 1) + (i >> 2);
            const int col = (16 * (grp & 1) + 4 * (i & 3)) * 2;
            const u32x2 lo = lds_read_tr16(kt + t0 * 64 + col);
            const u32x2 hi = lds_read_tr16(kt + (t0 + 8) * 64 + col);
            ka[hf] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    };
    // per-token scalars pass between the lanes through the wave's two LDS rows (fences: see the dz pass)
    auto put_rows = [&](float r0, float r1) {
        asm volatile("" ::: "memory");
        if (g2 == 0) {
            rb[c32] = r0;
            rb[32 + c32] = r1;
        }
        asm volatile("" ::: "memory");
    };
    auto read_row = [&](int which) {
        f32x16 o;
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(rb + 32 * which + 8 * j + 4 * g2);
            o[4 * j] = t[0]; o[4 * j + 1] = t[1]; o[4 * j + 2] = t[2]; o[4 * j + 3] = t[3];
        }
        asm volatile("" ::: "memory");
        return o;
    };
    // 8 + 8 packed bf16 of a token's row times a per-lane factor
    auto scale_rows = [&](u32x4 (&r)[2], float f) {
        r[0] = scale8_cvt(r[0], f);
        r[1] = scale8_cvt(r[1], f);
    };

    // A operand of the product with the per-latent scalars: k-slots ((eR delta) head, tail, head, 1, 1, 0, 0, 0) of the
    // lane's token in the lower half of the wave, zeros in the upper half
    auto extra_a = [&](float x) {
        const float xh = bf16_head(x);
        const u32x4 o = {pack2(xh, x - xh), pack2(xh, 1.f), pack2(1.f, 0.f), 0u};
        return g2 == 0 ? o : zero4();
    };

    f32x16 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = zero16();

    if (fast && n_full > 0) {
        u32x4 kb[2], vb[2], yb[2], kn[2], vn[2], yn[2];
        float rn, dn;                               // rho and delta of this lane's token in the next pass
        load_a(k, a.ks[2], first, kb);
        load_a(v, a.vs[2], first, vb);
        load_a(dy, a.dys[2], first, yb);
        rn = rho[min(first + c32, n_last)];
        dn = dlt[min(first + c32, n_last)];
        u32x4 ka[2] = {zero4(), zero4()};
        u32x4 pb[2] = {zero4(), zero4()};           // dS' of the previous slot (none yet: zeros)
        // latent operands of tile 0 (and its scores' operands), in registers one slot before their use from here on
        u32x4 q0 = qb[lane], q1 = qb[64 + lane];
        u32x4 od0 = dzb[lane], od1 = dzb[64 + lane], oz0 = zb[lane], oz1 = zb[64 + lane], ox = xb[lane];
        int n0 = first;
#pragma unroll 1
        for (int p = 0; p < n_full; ++p, n0 += 128) {
            // this pass: eR of the lane's token on its dY row, the row vector eR delta through LDS, K rows into the tile
            const float er = fast_exp2(lmax2 - rn * kLog2e);
            scale_rows(yb, er);
            const u32x4 xa = extra_a(er * dn);
            // the previous pass's last value product still reads the tile through ka: issue it before the tile changes
            acc[MT - 1] = mma32(ka[0], pb[0], acc[MT - 1]);
            acc[MT - 1] = mma32(ka[1], pb[1], acc[MT - 1]);
            put_k(kb);
            read_kt(ka);
            // the next pass's rows (the last pass requests rows of the range again, unused)
            load_a(k, a.ks[2], n0 + 128, kn);
            load_a(v, a.vs[2], n0 + 128, vn);
            load_a(dy, a.dys[2], n0 + 128, yn);
            rn = rho[min(n0 + 128 + c32, n_last)];
            dn = dlt[min(n0 + 128 + c32, n_last)];
            pb[0] = zero4();
            pb[1] = zero4();

            // (latent operands: each register is reloaded for the tile after next as soon as a product has consumed it)
            f32x16 sc = mma32(kb[0], q0, zero16());
            FLARE_FENCE();
            q0 = qb[2 * 64 + lane];
            FLARE_FENCE();
            sc = mma32(kb[1], q1, sc);
            FLARE_FENCE();
            q1 = qb[3 * 64 + lane];
            auto slot = [&](auto s_c) {
                constexpr int S = decltype(s_c)::value;
                constexpr int PREV = (S + MT - 1) % MT;
                constexpr int NX = (S + 1) % MT;        // tile whose g operands are requested in this slot
                constexpr int NQ = (S + 2) % MT;        // tile whose q operands are requested in this slot
                // g of this tile: five products on one accumulator, the exponentials run under them
                f32x16 g = mma32(xa, ox, zero16());
                FLARE_FENCE();
                ox = xb[NX * 64 + lane];
                f32x4 e0 = exp_quarter<0>(sc);
                FLARE_FENCE();
                g = mma32(vb[0], od0, g);
                FLARE_FENCE();
                od0 = dzb[(2 * NX) * 64 + lane];
                f32x4 e1 = exp_quarter<1>(sc);
                FLARE_FENCE();
                g = mma32(vb[1], od1, g);
                FLARE_FENCE();
                od1 = dzb[(2 * NX + 1) * 64 + lane];
                f32x4 e2 = exp_quarter<2>(sc);
                FLARE_FENCE();
                g = mma32(yb[0], oz0, g);
                FLARE_FENCE();
                oz0 = zb[(2 * NX) * 64 + lane];
                f32x4 e3 = exp_quarter<3>(sc);
                FLARE_FENCE();
                g = mma32(yb[1], oz1, g);
                FLARE_FENCE();
                oz1 = zb[(2 * NX + 1) * 64 + lane];
                // the previous slot's value product and the next tile's scores, while g finishes
                f32x16 sn = sc;
                if constexpr (S > 0) {
                    acc[PREV] = mma32(ka[0], pb[0], acc[PREV]);
                    FLARE_FENCE();
                }
                if constexpr (S + 1 < MT) {
                    sn = mma32(kb[0], q0, zero16());
                    FLARE_FENCE();
                    q0 = qb[(2 * NQ) * 64 + lane];
                    FLARE_FENCE();
                }
                if constexpr (S > 0) {
                    acc[PREV] = mma32(ka[1], pb[1], acc[PREV]);
                    FLARE_FENCE();
                }
                if constexpr (S + 1 < MT) {
                    sn = mma32(kb[1], q1, sn);
                    FLARE_FENCE();
                    q1 = qb[(2 * NQ + 1) * 64 + lane];
                    FLARE_FENCE();
                }
                // dS' = exp2(S) g (g with its two per-latent terms), packed as the B operands of the value product
                u32x4 pc[2];
                const f32x4 ex[4] = {e0, e1, e2, e3};
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    float o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[i] = ex[qd][i] * g[4 * qd + i];
                    pc[qd >> 1][2 * (qd & 1)] = pack2(o[0], o[1]);
                    pc[qd >> 1][2 * (qd & 1) + 1] = pack2(o[2], o[3]);
                }
                pb[0] = pc[0];
                pb[1] = pc[1];
                sc = sn;
            };
            static_for<0, MT>(slot);
            kb[0] = kn[0]; kb[1] = kn[1];
            vb[0] = vn[0]; vb[1] = vn[1];
            yb[0] = yn[0]; yb[1] = yn[1];
        }
        acc[MT - 1] = mma32(ka[0], pb[0], acc[MT - 1]);
        acc[MT - 1] = mma32(ka[1], pb[1], acc[MT - 1]);
    }

    // One pass without pipelining: the shorter last pass of a range, and every pass of a (b,h) in the general form.
    auto plain_pass = [&](auto fast_c, int n0, int valid) {
        constexpr bool FAST = decltype(fast_c)::value;
        u32x4 kb[2], vb[2], yb[2], ka[2];
        load_a(k, a.ks[2], n0, kb);
        load_a(v, a.vs[2], n0, vb);
        load_a(dy, a.dys[2], n0, yb);
        const float r2 = rho[min(n0 + c32, n_last)] * kLog2e, dl = dlt[min(n0 + c32, n_last)];
        f32x16 row0 = zero16(), row1 = zero16();
        u32x4 xa = zero4();
        if constexpr (FAST) {
            const float er = fast_exp2(lmax2 - r2);
            scale_rows(yb, er);
            xa = extra_a(er * dl);
        } else {
            put_rows(-r2, -dl);
            row0 = read_row(0);                     // -rho2
            row1 = read_row(1);                     // -delta
        }
        put_k(kb);
        read_kt(ka);
        bool ok[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) ok[r] = 8 * (r >> 2) + 4 * g2 + (r & 3) < valid;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const u32x4 q0 = qb[(2 * mt) * 64 + lane], q1 = qb[(2 * mt + 1) * 64 + lane];
            const u32x4 d0 = dzb[(2 * mt) * 64 + lane], d1 = dzb[(2 * mt + 1) * 64 + lane];
            const u32x4 z0 = zb[(2 * mt) * 64 + lane], z1 = zb[(2 * mt + 1) * 64 + lane];
            f32x16 s = mma32(kb[0], q0, zero16());
            s = mma32(kb[1], q1, s);
            float o[16];
            if constexpr (FAST) {
                f32x16 g = mma32(xa, xb[mt * 64 + lane], zero16());
                g = mma32(vb[0], d0, g);
                g = mma32(vb[1], d1, g);
                g = mma32(yb[0], z0, g);
                g = mma32(yb[1], z1, g);
#pragma unroll
                for (int r = 0; r < 16; ++r) o[r] = fast_exp2(s[r]) * g[r];
            } else {
                f32x16 g1 = mma32(vb[0], d0, zero16());
                g1 = mma32(vb[1], d1, g1);
                f32x16 g2v = mma32(yb[0], z0, row1);        // <dy_n, z_m> - delta_n
                g2v = mma32(yb[1], z1, g2v);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    o[r] = fast_exp2(s[r] - l2m[mt]) * (g1[r] - dm[mt]) + fast_exp2(s[r] + row0[r]) * g2v[r];
            }
            u32x4 p[2];
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e >> 2][e & 3] = pack2(ok[2 * e] ? o[2 * e] : 0.f, ok[2 * e + 1] ? o[2 * e + 1] : 0.f);
            acc[mt] = mma32(ka[0], p[0], acc[mt]);
            acc[mt] = mma32(ka[1], p[1], acc[mt]);
        }
    };
    if (fast) {
        if (tail_valid > 0) plain_pass(std::true_type{}, tail0, tail_valid);
    } else {
#pragma unroll 1
        for (int n0 = first; n0 < n_end; n0 += 128) plain_pass(std::false_type{}, n0, min(32, n_end - n0));
    }

    // the one-exponential form left out the per-latent constant of the gather's weights
    if (fast) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] *= fast_exp2(-l2m[mt]);
    }

    // ---- the four waves' sums meet in LDS: (w0 + w2) + (w1 + w3) --------------------------------------------
    constexpr int kSlotB = MT * 4 * 64 * 16;
    auto publish = [&](int slot_i) {
        f32x4* z4 = reinterpret_cast<f32x4*>(smem32q + slot_i * kSlotB);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                z4[(mt * 4 + j) * 64 + lane] = f32x4{acc[mt][4 * j], acc[mt][4 * j + 1], acc[mt][4 * j + 2], acc[mt][4 * j + 3]};
    };
    auto absorb = [&](int slot_i) {
        const f32x4* z4 = reinterpret_cast<const f32x4*>(smem32q + slot_i * kSlotB);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 o = z4[(mt * 4 + j) * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[mt][4 * j + i] += o[i];
            }
    };
    __syncthreads();
    if (w >= 2) publish(w - 2);
    __syncthreads();
    if (w < 2) absorb(w);
    __syncthreads();
    if (w == 1) publish(0);
    __syncthreads();
    if (w == 0) {
        absorb(0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m_base + mt * 32 + c32;
            const int64_t row = (bh * a.n_splits + split) * a.M + m;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<f32x4*>(a.part + row * D + 8 * j + 4 * g2) =
                    f32x4{acc[mt][4 * j], acc[mt][4 * j + 1], acc[mt][4 * j + 2], acc[mt][4 * j + 3]};
        }
    }
}

template <int MT>
constexpr size_t dq32_lds()
{
    const size_t main_b = (size_t)3 * MT * 2048 + MT * 1024 + 4 * 2048 + 4 * 256;
    const size_t red_b = 2 * ((size_t)MT * 4 * 64 * 16);
    return main_b > red_b ? main_b : red_b;
}

template <int MT>
hipError_t dq32_launch(const MixerBwdArgs& a, hipStream_t st)
{
    auto kern = bwd_dq32_kernel<MT>;
    constexpr size_t lds = dq32_lds<MT>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    dim3 grid((a.n_splits + 7) / 8 * 8 * (a.M / (32 * MT)), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a);
    return hipGetLastError();
}

// =====================================================================================
// token pass: dv_n = sum_m A[m,n] dz_m,  dk_n = s sum_m dS[m,n] q_m
// =====================================================================================
// The forward scatter's shape (mixer_mfma32.hip): one workgroup = 8 independent waves sharing the latent operands in
// LDS; a wave pass covers one column tile of 32 tokens against all M = 32 KS latents, 32 at a time.  Tiles have rows =
// latents and the lane's column = its token, so tokens never meet each other's numbers (rows past the range repeat the
// last row and are not stored).  Per (latent step, token tile), in the unshifted one-exponential form
// (bwd_unshifted_form; the other (b,h) are left to bwd_tok_kernel of mixer_bwd_mfma.hip, launched behind this one):
//   S = q k^T,   g = dz v^T + (eL z)(eR dy)^T + (-eL, -Delta)((eR delta), 1)^T   in one accumulator chain (5 products),
//   A' = exp2(S),  dS' = A' g,   dv^T += (c dz)^T A',   dk^T += (s c q)^T dS'      with c_m = exp2(-L2_m)
// The constant c_m of the gather's weights, a row factor of the tile, rides on the two operand sets that contract over
// the latents.  Two vector instructions per score (exponential, multiply) and a pack of each of A' and dS'.
constexpr int kTok32Waves = 8;

template <int KS>
__global__ __launch_bounds__(64 * kTok32Waves, 1) void bwd_tok32_kernel(MixerBwdArgs a, int tokens_per_wg)
{
    constexpr int D = 32, M = 32 * KS, NTH = 64 * kTok32Waves;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem32t[];
    // qa, dza, zza [mt][kd][lane]: A operands of the score-like products, latent 32 mt + c32, d = 16 kd + 8 g2 .. + 7
    // dzt, qt [mt][hf][lane]: A operands of the products over the latents, row c32 = output column
    //     d(c32) = 16 ((c32 >> 2) & 1) + 4 (c32 >> 3) + (c32 & 3), k-slot e = latent 32 mt + 16 hf + 8 (e / 4) + 4 g2 + e % 4
    // xa [mt][lane]: A operand of the product with the per-latent scalars (-eL head, -eL head, -eL tail, -Delta head, -Delta tail)
    u32x4* qa = reinterpret_cast<u32x4*>(smem32t);
    u32x4* dza = qa + KS * 128;
    u32x4* zza = dza + KS * 128;
    u32x4* dzt = zza + KS * 128;
    u32x4* qt = dzt + KS * 128;
    u32x4* xa = qt + KS * 128;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g2 = lane >> 5, c32 = lane & 31;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;
    float lmax2;
    if (!bwd_unshifted_form(a, bh, lane, lmax2)) return;       // uniform over the workgroup

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint16_t* dy = (const uint16_t*)a.dy + b * a.dys[0] + h * a.dys[1];
    uint16_t* dk = (uint16_t*)a.dk + b * a.dks[0] + h * a.dks[1];
    uint16_t* dv = (uint16_t*)a.dv + b * a.dvs[0] + h * a.dvs[1];
    const float* z = a.z + bh * M * D;
    const float* dz = a.dz + bh * M * D;
    const float* lse_lat = a.lse_lat + bh * M;
    const float* rho = a.lse_tok + bh * a.N;
    const float* dlt = a.delta_tok + bh * a.N;

    for (int idx = tid; idx < KS * 128; idx += NTH) {
        const int ln = idx & 63, kd = (idx >> 6) & 1, mt = idx >> 7;
        const int m = 32 * mt + (ln & 31), ch = 2 * kd + (ln >> 5);
        qa[idx] = scale8(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2);
        dza[idx] = pack8f(dz + (int64_t)m * D + ch * 8, 1.f);
        zza[idx] = pack8f(z + (int64_t)m * D + ch * 8, fast_exp2(lse_lat[m] * kLog2e - lmax2));
    }
    for (int idx = tid; idx < KS * 128; idx += NTH) {
        const int ln = idx & 63, hf = (idx >> 6) & 1, mt = idx >> 7;
        const int r = ln & 31, gg = ln >> 5;
        const int d = 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
        u32x4 o1, o2;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            const int e = 2 * e2;
            const int m0 = 32 * mt + 16 * hf + 8 * (e >> 2) + 4 * gg + (e & 3);
            const float c0 = fast_exp2(-lse_lat[m0] * kLog2e), c1 = fast_exp2(-lse_lat[m0 + 1] * kLog2e);
            o1[e2] = pack2(dz[(int64_t)m0 * D + d] * c0, dz[(int64_t)(m0 + 1) * D + d] * c1);
            o2[e2] = pack2(__uint_as_float(uint32_t(q[(int64_t)m0 * a.qs[2] + d]) << 16) * (a.scale * c0),
                           __uint_as_float(uint32_t(q[(int64_t)(m0 + 1) * a.qs[2] + d]) << 16) * (a.scale * c1));
        }
        dzt[idx] = o1;
        qt[idx] = o2;
    }
    for (int idx = tid; idx < KS * 64; idx += NTH) {
        const int ln = idx & 63, mt = idx >> 6;
        const int m = 32 * mt + (ln & 31);
        const float el = fast_exp2(lse_lat[m] * kLog2e - lmax2), de = a.delta_lat[bh * M + m];
        const float el_h = bf16_head(el), de_h = bf16_head(de);
        const u32x4 o = {pack2(-el_h, -el_h), pack2(-(el - el_h), -de_h), pack2(-(de - de_h), 0.f), 0u};
        xa[idx] = (ln >> 5) == 0 ? o : zero4();
    }
    __syncthreads();

    const int wg_n0 = blockIdx.x * tokens_per_wg;
    const int wg_n1 = min(a.N, wg_n0 + tokens_per_wg);
    const int n_lastrow = max(wg_n1 - 1, 0);
    constexpr int kStride = kTok32Waves * 32;
    int t0 = wg_n0 + w * 32;
    if (t0 >= wg_n1) return;

    // rows of the lane's token as B operands: d = 16 kd + 8 g2 .. + 7
    auto load_b = [&](const uint16_t* base, int64_t stride, int n0, u32x4 (&dst)[2]) {
        const uint16_t* r = base + (int64_t)min(n0 + c32, n_lastrow) * stride + g2 * 8;
        dst[0] = load16_stream(r);
        dst[1] = load16_stream(r + 16);
    };
    u32x4 kn[2], vn[2], yn[2];
    float rn, dn;
    load_b(k, a.ks[2], t0, kn);
    load_b(v, a.vs[2], t0, vn);
    load_b(dy, a.dys[2], t0, yn);
    rn = rho[min(t0 + c32, n_lastrow)];
    dn = dlt[min(t0 + c32, n_lastrow)];
    // latent operands of step 0, in registers one slot before their use from here on
    u32x4 oq0 = qa[lane], oq1 = qa[64 + lane];
    u32x4 od0 = dza[lane], od1 = dza[64 + lane], oz0 = zza[lane], oz1 = zza[64 + lane], ox = xa[lane];
    u32x4 ot0 = dzt[lane], ot1 = dzt[64 + lane], ou0 = qt[lane], ou1 = qt[64 + lane];

#pragma unroll 1
    for (; t0 < wg_n1; t0 += kStride) {
        u32x4 kb[2] = {kn[0], kn[1]}, vb[2] = {vn[0], vn[1]}, yb[2] = {yn[0], yn[1]};
        const float er = fast_exp2(lmax2 - rn * kLog2e);
        const float x = er * dn;
        // the next pass's rows (the last pass requests rows of the range again, unused)
        const int tn = t0 + kStride;
        load_b(k, a.ks[2], tn, kn);
        load_b(v, a.vs[2], tn, vn);
        load_b(dy, a.dys[2], tn, yn);
        rn = rho[min(tn + c32, n_lastrow)];
        dn = dlt[min(tn + c32, n_lastrow)];
        yb[0] = scale8_cvt(yb[0], er);
        yb[1] = scale8_cvt(yb[1], er);
        // B operand of the product with the per-latent scalars: k-slots ((eR delta) head, tail, head, 1, 1, 0, 0, 0)
        const float xh = bf16_head(x);
        const u32x4 xfull = {pack2(xh, x - xh), pack2(xh, 1.f), pack2(1.f, 0.f), 0u};
        const u32x4 xbk = g2 == 0 ? xfull : zero4();

        f32x16 adv = zero16(), adk = zero16();
        u32x4 pa[2] = {zero4(), zero4()}, pd[2] = {zero4(), zero4()};
        f32x16 sc = mma32(oq0, kb[0], zero16());
        FLARE_FENCE();
        oq0 = qa[2 * 64 + lane];
        FLARE_FENCE();
        sc = mma32(oq1, kb[1], sc);
        FLARE_FENCE();
        oq1 = qa[3 * 64 + lane];
        auto slot = [&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            constexpr int NX = (S + 1) % KS;        // step whose g operands are requested in this slot
            constexpr int NQ = (S + 2) % KS;        // step whose q operands are requested in this slot
            f32x16 g = mma32(ox, xbk, zero16());
            FLARE_FENCE();
            ox = xa[NX * 64 + lane];
            f32x4 e0 = exp_quarter<0>(sc);
            FLARE_FENCE();
            g = mma32(od0, vb[0], g);
            FLARE_FENCE();
            od0 = dza[(2 * NX) * 64 + lane];
            f32x4 e1 = exp_quarter<1>(sc);
            FLARE_FENCE();
            g = mma32(od1, vb[1], g);
            FLARE_FENCE();
            od1 = dza[(2 * NX + 1) * 64 + lane];
            f32x4 e2 = exp_quarter<2>(sc);
            FLARE_FENCE();
            g = mma32(oz0, yb[0], g);
            FLARE_FENCE();
            oz0 = zza[(2 * NX) * 64 + lane];
            f32x4 e3 = exp_quarter<3>(sc);
            FLARE_FENCE();
            g = mma32(oz1, yb[1], g);
            FLARE_FENCE();
            oz1 = zza[(2 * NX + 1) * 64 + lane];
            // the previous step's products over the latents and the next step's scores, while g finishes
            f32x16 sn = sc;
            if constexpr (S > 0) {
                adv = mma32(ot0, pa[0], adv);
                FLARE_FENCE();
                ot0 = dzt[(2 * S) * 64 + lane];
                FLARE_FENCE();
                adk = mma32(ou0, pd[0], adk);
                FLARE_FENCE();
                ou0 = qt[(2 * S) * 64 + lane];
                FLARE_FENCE();
            }
            if constexpr (S + 1 < KS) {
                sn = mma32(oq0, kb[0], zero16());
                FLARE_FENCE();
                oq0 = qa[(2 * NQ) * 64 + lane];
                FLARE_FENCE();
            }
            if constexpr (S > 0) {
                adv = mma32(ot1, pa[1], adv);
                FLARE_FENCE();
                ot1 = dzt[(2 * S + 1) * 64 + lane];
                FLARE_FENCE();
                adk = mma32(ou1, pd[1], adk);
                FLARE_FENCE();
                ou1 = qt[(2 * S + 1) * 64 + lane];
                FLARE_FENCE();
            }
            if constexpr (S + 1 < KS) {
                sn = mma32(oq1, kb[1], sn);
                FLARE_FENCE();
                oq1 = qa[(2 * NQ + 1) * 64 + lane];
                FLARE_FENCE();
            }
            // A' and dS' = A' g, packed as the B operands of the products over the latents
            const f32x4 ex[4] = {e0, e1, e2, e3};
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                pa[qd >> 1][2 * (qd & 1)] = pack2(ex[qd][0], ex[qd][1]);
                pa[qd >> 1][2 * (qd & 1) + 1] = pack2(ex[qd][2], ex[qd][3]);
                pd[qd >> 1][2 * (qd & 1)] = pack2(ex[qd][0] * g[4 * qd], ex[qd][1] * g[4 * qd + 1]);
                pd[qd >> 1][2 * (qd & 1) + 1] = pack2(ex[qd][2] * g[4 * qd + 2], ex[qd][3] * g[4 * qd + 3]);
            }
            sc = sn;
        };
        static_for<0, KS>(slot);
        // the last step's products; their operand registers go back to step 0 for the next pass
        adv = mma32(ot0, pa[0], adv);
        adk = mma32(ou0, pd[0], adk);
        adv = mma32(ot1, pa[1], adv);
        adk = mma32(ou1, pd[1], adk);
        ot0 = dzt[lane];
        ot1 = dzt[64 + lane];
        ou0 = qt[lane];
        ou1 = qt[64 + lane];

        // lane (token c32, g2) owns d = 16 g2 .. 16 g2 + 15 of both gradients (register 4 j + i: d = 16 g2 + 4 j + i)
        const int n = t0 + c32;
        if (n < wg_n1) {
            uint32_t o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = pack2(adk[2 * e], adk[2 * e + 1]);
            uint16_t* pk = dk + (int64_t)n * a.dks[2] + 16 * g2;
            *reinterpret_cast<u32x4*>(pk) = u32x4{o[0], o[1], o[2], o[3]};
            *reinterpret_cast<u32x4*>(pk + 8) = u32x4{o[4], o[5], o[6], o[7]};
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = pack2(adv[2 * e], adv[2 * e + 1]);
            uint16_t* pv = dv + (int64_t)n * a.dvs[2] + 16 * g2;
            *reinterpret_cast<u32x4*>(pv) = u32x4{o[0], o[1], o[2], o[3]};
            *reinterpret_cast<u32x4*>(pv + 8) = u32x4{o[4], o[5], o[6], o[7]};
        }
    }
}

template <int KS>
hipError_t tok32_launch(const MixerBwdArgs& a, hipStream_t st)
{
    auto kern = bwd_tok32_kernel<KS>;
    const size_t lds = (size_t)KS * (5 * 2048 + 1024);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    // one workgroup per compute unit, ranges a multiple of its eight waves' 32-token passes
    const int64_t per_bh = (device_cus() + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H);
    int64_t tpw = (a.N + per_bh - 1) / per_bh;
    tpw = ((tpw + 255) / 256) * 256;
    dim3 grid((unsigned)((a.N + tpw - 1) / tpw), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(64 * kTok32Waves), lds, st, a, (int)tpw);
    return hipGetLastError();
}

// LDS of a workgroup: the latent operands, four dY tiles, four rows of shifts and four maxima in the token loop; two
// publishing slots afterwards
template <int MT>
constexpr size_t dz32_lds()
{
    const size_t main_b = (size_t)MT * 2048 + 4 * 2048 + 4 * 128 + 16;
    const size_t red_b = 2 * ((size_t)MT * 4 * 64 * 16);
    return main_b > red_b ? main_b : red_b;
}

template <int MT>
hipError_t dz32_launch(const MixerBwdArgs& a, hipStream_t st)
{
    auto kern = bwd_dz32_kernel<MT>;
    constexpr size_t lds = dz32_lds<MT>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    dim3 grid(a.n_splits * (a.M / (32 * MT)), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a);
    return hipGetLastError();
}

}  // namespace

// bf16, D = 32, latent counts that are multiples of 64 (256, 128 or 64 latents per workgroup)
bool bwd_dz32_supported(int dtype, int M, int D)
{
    return dtype == 1 && D == 32 && M >= 64 && M % 64 == 0;
}

// bf16, D = 32, 64, 128 or 256 latents (the six operand sets of more do not fit the LDS)
bool bwd_tok32_supported(int dtype, int M, int D)
{
    return dtype == 1 && D == 32 && (M == 64 || M == 128 || M == 256);
}

hipError_t launch_bwd_tok32(const MixerBwdArgs& a, hipStream_t st)
{
    switch (a.M) {
        case 64:  return tok32_launch<2>(a, st);
        case 128: return tok32_launch<4>(a, st);
        case 256: return tok32_launch<8>(a, st);
        default:  return hipErrorInvalidValue;
    }
}

// latent blocks of a dq-pass workgroup grid (128 latents per workgroup, 64 where M is not a multiple of 128)
int bwd_dq32_mblocks(int M) { return M % 128 == 0 ? M / 128 : M / 64; }

hipError_t launch_bwd_dq32(const MixerBwdArgs& a, hipStream_t st)
{
    return a.M % 128 == 0 ? dq32_launch<4>(a, st) : dq32_launch<2>(a, st);
}

// `a` carries the dz pass's own split of the token axis in n_splits / tokens_per_split
hipError_t launch_bwd_dz32(const MixerBwdArgs& a, hipStream_t st)
{
    return a.M % 256 == 0 ? dz32_launch<8>(a, st) : a.M % 128 == 0 ? dz32_launch<4>(a, st) : dz32_launch<2>(a, st);
}

}  // namespace flare
