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
// (scatter) or by the addresses of the LDS transpose reads (gather).  Both kernels are token parallel: a wave
// streams its own tokens' K rows straight from global memory into matrix operands and shares nothing but the
// latent operands in LDS with the other waves, so there is no barrier in either token loop.
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
#include "mfma32.hpp"

namespace flare {

namespace {

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
// gather: z = softmax_n(s q k^T) v, token parallel inside a workgroup
// =====================================================================================
// One workgroup = 4 waves that own the same 32 MT latents and different tokens: wave w takes the 32-token passes
// w, w + 4, w + 8, ... of the workgroup's token range.  Score tile: rows = tokens (A = K rows, straight from global
// memory, one lane per token), columns = latents (B = Q, read from LDS where it is written once in operand order).
// The sixteen accumulators of a score tile, exponentiated and packed, are the two B operands of the value product;
// its A operand V^T comes from a wave-private LDS tile through the transposing read.  Nothing in the token loop is
// shared between waves: no barrier.  The pipeline unit is a slot = (pass, latent tile): the matrix pipe computes the
// scores of slot s + 1 and the value product of slot s - 1 while the vector ALU exponentiates slot s; the slots of
// consecutive passes form one sequence.  K and V rows of the next pass are requested at the start of a pass.
// At the end the four waves' sums meet in LDS and the workgroup writes one partial.
template <int MT>
__global__ __launch_bounds__(256, 2) void gather32_kernel(MixerArgs a)
{
    constexpr int D = 32;
    static_assert(MT >= 2, "at least two latent tiles per wave");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem32g[];
    u32x4* qb = reinterpret_cast<u32x4*>(smem32g);              // [MT][2][64]: B operands of the score product

    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g2 = lane >> 5, c32 = lane & 31;
    uint8_t* vb = smem32g + MT * 2048 + w * 2048;               // this wave's V tile: 32 rows of 64 bytes
    const int mblocks = a.M / (32 * MT);
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const int m_base = mb * 32 * MT;

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

    // K rows of a pass as A operands: lane (token c32, g2) holds d = 16 kd + 8 g2 .. + 7.  V rows as they are
    // written to the LDS tile: lane l holds the 16-byte chunk l % 4 of row 16 j + l / 4.
    // Rows past the end of the range repeat its last row (their probabilities are set to zero where they are used).
    auto load_k = [&](int n0, u32x4 (&dst)[2]) {
        const uint16_t* kr = k + (int64_t)min(n0 + c32, n_last) * a.ks[2] + g2 * 8;
        dst[0] = load16_stream(kr);
        dst[1] = load16_stream(kr + 16);
    };
    auto load_v = [&](int n0, u32x4 (&dst)[2]) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            dst[j] = load16_stream(v + (int64_t)min(n0 + 16 * j + (lane >> 2), n_last) * a.vs[2] + (lane & 3) * 8);
    };
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

    float shift[MT];
    f32x16 zacc[MT];
    float lsum[MT];       // this lane's share of the denominators (its 16 tokens of every pass)

    // ---- optimistic passes: no softmax shift ---------------------------------------------------------------
    {
        // Denominators: v_mfma_f32_4x4x4_16B_bf16 with a row selector as A adds the four probabilities a lane holds in
        // two registers into register r of the accumulator (A row r = ones, the other rows zeros), so one f32x4 serves
        // four latent tiles.
        constexpr int ND = (MT + 3) / 4;
        f32x4 dsum4[ND];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            shift[mt] = 0.f;
            zacc[mt] = zero16();
            lsum[mt] = 0.f;
        }
#pragma unroll
        for (int i = 0; i < ND; ++i) dsum4[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (n_full > 0) {
            u32x2 sel[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t o = (lane & 3) == r ? 0x3f803f80u : 0u;
                sel[r] = u32x2{o, o};
            }
            // uniform row bases that advance by a pass, per-lane byte offsets inside a pass (no clamps: full passes only)
            const char* kbase = reinterpret_cast<const char*>(k + (int64_t)first * a.ks[2]);
            const char* vbase0 = reinterpret_cast<const char*>(v + (int64_t)first * a.vs[2]);
            const char* vbase1 = reinterpret_cast<const char*>(v + (int64_t)(first + 16) * a.vs[2]);
            const uint32_t koff = (uint32_t)((c32 * a.ks[2] + g2 * 8) * 2);
            const uint32_t voff = (uint32_t)(((lane >> 2) * a.vs[2] + (lane & 3) * 8) * 2);
            const int64_t kstep = 256 * a.ks[2], vstep = 256 * a.vs[2];       // bytes per 128 rows
            auto ld_k = [&](u32x4 (&dst)[2]) {
                dst[0] = load16_stream(kbase + koff);
                dst[1] = load16_stream(kbase + koff + 32);
            };
            auto ld_v = [&](u32x4 (&dst)[2]) {
                dst[0] = load16_stream(vbase0 + voff);
                dst[1] = load16_stream(vbase1 + voff);
            };
            u32x4 kb[2], kn[2], vr[2];
            u32x4 va[2] = {zero4(), zero4()};
            u32x4 pb[2] = {zero4(), zero4()};      // probabilities of the previous slot (none yet: zeros, met by zero values)
            u32x4 qreg[2];
            ld_k(kb);
            ld_v(vr);
            qreg[0] = qb[lane];
            qreg[1] = qb[64 + lane];
            f32x16 sc = mma32(kb[0], qreg[0], zero16());
            sc = mma32(kb[1], qreg[1], sc);
            qreg[0] = qb[2 * 64 + lane];
            qreg[1] = qb[3 * 64 + lane];

            auto den = [&](auto prev_c, auto q_c) {
                constexpr int PREV = decltype(prev_c)::value, QQ = decltype(q_c)::value;
                dsum4[PREV >> 2] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
                    __builtin_bit_cast(s16x4, sel[PREV & 3]),
                    __builtin_bit_cast(s16x4, u32x2{pb[QQ >> 1][2 * (QQ & 1)], pb[QQ >> 1][2 * (QQ & 1) + 1]}), dsum4[PREV >> 2], 0, 0, 0);
            };
            using Q0 = std::integral_constant<int, 0>;
            using Q1 = std::integral_constant<int, 1>;
            using Q2 = std::integral_constant<int, 2>;
            using Q3 = std::integral_constant<int, 3>;

            // One slot: exponentials of the current scores (sc); scores of the next slot (latent tile (S + 1) % MT, of the
            // next pass's rows in the last slot); value product and denominators of the previous slot.  The latent
            // operands of the slot after the next one are requested as soon as a product has consumed its register.
            auto slot = [&](auto s_c) {
                constexpr int S = decltype(s_c)::value;
                constexpr bool LAST = S + 1 == MT;
                using PREV = std::integral_constant<int, (S + MT - 1) % MT>;
                constexpr int QF = (S + 2) % MT;
                const u32x4 kx0 = LAST ? kn[0] : kb[0], kx1 = LAST ? kn[1] : kb[1];
                f32x16 sn;
                u32x4 pc[2];
                f32x4 ex;
                // quarter 0
                sn = mma32(kx0, qreg[0], zero16());
                FLARE_FENCE();
                qreg[0] = qb[(2 * QF) * 64 + lane];
                ex = exp_quarter<0>(sc);
                FLARE_FENCE();
                den(PREV{}, Q0{});
                FLARE_FENCE();
                pack_quarter<0>(ex, pc);
                FLARE_FENCE();
                // quarter 1
                zacc[PREV::value] = mma32(va[0], pb[0], zacc[PREV::value]);
                FLARE_FENCE();
                ex = exp_quarter<1>(sc);
                FLARE_FENCE();
                den(PREV{}, Q1{});
                FLARE_FENCE();
                pack_quarter<1>(ex, pc);
                FLARE_FENCE();
                // quarter 2
                sn = mma32(kx1, qreg[1], sn);
                FLARE_FENCE();
                qreg[1] = qb[(2 * QF + 1) * 64 + lane];
                ex = exp_quarter<2>(sc);
                FLARE_FENCE();
                den(PREV{}, Q2{});
                FLARE_FENCE();
                pack_quarter<2>(ex, pc);
                FLARE_FENCE();
                // quarter 3
                zacc[PREV::value] = mma32(va[1], pb[1], zacc[PREV::value]);
                FLARE_FENCE();
                if constexpr (S == 0) read_v(va);      // this pass's V^T, after the last product with the previous pass's
                ex = exp_quarter<3>(sc);
                FLARE_FENCE();
                den(PREV{}, Q3{});
                FLARE_FENCE();
                pack_quarter<3>(ex, pc);
                FLARE_FENCE();
                pb[0] = pc[0];
                pb[1] = pc[1];
                sc = sn;
            };

            asm volatile("" ::"v"(kb[0]), "v"(kb[1]));
#pragma unroll 1
            for (int p = 0; p < n_full; ++p) {
                put_v(vr);
                const bool more = p + 1 < n_full;       // the last pass requests its own rows again (unused)
                kbase += more ? kstep : 0;
                vbase0 += more ? vstep : 0;
                vbase1 += more ? vstep : 0;
                ld_k(kn);
                ld_v(vr);
                static_for<0, MT>(slot);
                kb[0] = kn[0];
                kb[1] = kn[1];
            }
            // drain: the last slot's value product and denominators
            zacc[MT - 1] = mma32(va[0], pb[0], zacc[MT - 1]);
            zacc[MT - 1] = mma32(va[1], pb[1], zacc[MT - 1]);
            using PL = std::integral_constant<int, MT - 1>;
            den(PL{}, Q0{});
            den(PL{}, Q1{});
            den(PL{}, Q2{});
            den(PL{}, Q3{});
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) lsum[mt] = dsum4[mt >> 2][mt & 3];
    }

    // one pass without pipelining: the shorter last pass of a range (`valid` tokens), and every pass of a wave
    // that repeats its range with a running maximum per latent (EXACT)
    auto plain_pass = [&](auto exact_c, int n0, int valid) {
        constexpr bool EXACT = decltype(exact_c)::value;
        u32x4 kb[2], vr[2], va[2];
        load_k(n0, kb);
        load_v(n0, vr);
        put_v(vr);
        read_v(va);
        bool ok[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) ok[r] = 8 * (r >> 2) + 4 * g2 + (r & 3) < valid;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const u32x4 q0 = qb[(2 * mt) * 64 + lane], q1 = qb[(2 * mt + 1) * 64 + lane];
            f32x16 s = mma32(kb[0], q0, zero16());
            s = mma32(kb[1], q1, s);
            float nc = 0.f;
            if (EXACT) {
                float mx = kNegBig;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (ok[r]) mx = fmaxf(mx, s[r]);
                mx = max_xor32(mx);
                nc = fmaxf(shift[mt], mx);
                const float al = fast_exp2(shift[mt] - nc);
                zacc[mt] *= al;
                lsum[mt] *= al;
                shift[mt] = nc;
            }
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
            lsum[mt] += tsum;
            zacc[mt] = mma32(va[0], p[0], zacc[mt]);
            zacc[mt] = mma32(va[1], p[1], zacc[mt]);
        }
    };
    if (tail_valid > 0) plain_pass(std::false_type{}, tail0, tail_valid);

    // validate: every denominator of this wave inside the safe range, numerators finite (and small enough for the
    // sum of four waves); a wave that fails repeats its own passes with a running maximum
    float lfull[MT];
    {
        bool bad = false;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float l = sum_xor32(lsum[mt]);
            lfull[mt] = l;
            bad = bad || !(l <= kLMax) || (first < n_end && !(l >= kLMin));
#pragma unroll
            for (int r = 0; r < 16; ++r) bad = bad || !(fabsf(zacc[mt][r]) <= 8.0e37f);
        }
        if (__any(bad)) {
            asm volatile("; exact pass" ::: "memory");
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                shift[mt] = kNegBig;
                zacc[mt] = zero16();
                lsum[mt] = 0.f;
            }
#pragma unroll 1
            for (int n0 = first; n0 < n_end; n0 += 128) plain_pass(std::true_type{}, n0, min(32, n_end - n0));
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) lfull[mt] = sum_xor32(lsum[mt]);
        }
    }

    // ---- the four waves' sums meet in LDS: (w0 + w2) + (w1 + w3) --------------------------------------------
    // slot layout: [MT * 4][64] f32x4 numerators, then [MT][64] shifts, [MT][64] sums
    constexpr int kSlotB = MT * 4 * 64 * 16 + 2 * MT * 64 * 4;
    auto publish = [&](int slot_i) {
        uint8_t* base = smem32g + slot_i * kSlotB;
        f32x4* z4 = reinterpret_cast<f32x4*>(base);
        float* sh = reinterpret_cast<float*>(base + MT * 4 * 64 * 16);
        float* ls = sh + MT * 64;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                z4[(mt * 4 + j) * 64 + lane] = f32x4{zacc[mt][4 * j], zacc[mt][4 * j + 1], zacc[mt][4 * j + 2], zacc[mt][4 * j + 3]};
            sh[mt * 64 + lane] = shift[mt];
            ls[mt * 64 + lane] = lfull[mt];
        }
    };
    auto absorb = [&](int slot_i) {
        const uint8_t* base = smem32g + slot_i * kSlotB;
        const f32x4* z4 = reinterpret_cast<const f32x4*>(base);
        const float* sh = reinterpret_cast<const float*>(base + MT * 4 * 64 * 16);
        const float* ls = sh + MT * 64;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float so = sh[mt * 64 + lane], lo = ls[mt * 64 + lane];
            const float ns = fmaxf(shift[mt], so);
            const float fa = fast_exp2(shift[mt] - ns), fb = fast_exp2(so - ns);
            lfull[mt] = lfull[mt] * fa + lo * fb;
            shift[mt] = ns;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 o = z4[(mt * 4 + j) * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; ++i) zacc[mt][4 * j + i] = zacc[mt][4 * j + i] * fa + o[i] * fb;
            }
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
        // partial for this split: shift (log2 units), sum, numerator, renormalised so that the sum has exponent 0
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float l = lfull[mt];
            int e = 0;
            if (l > 0.f) (void)frexpf(l, &e);
            const float scl = l > 0.f ? ldexpf(1.f, -e) : 0.f;
            const int m = m_base + mt * 32 + c32;
            const int64_t row = (((int64_t)b * a.H + h) * a.n_parts + split) * a.M + m;
            if (g2 == 0) {
                a.part_m[row] = l > 0.f ? shift[mt] + (float)e : kNegBig;
                a.part_l[row] = l * scl;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 o = {zacc[mt][4 * j] * scl, zacc[mt][4 * j + 1] * scl, zacc[mt][4 * j + 2] * scl, zacc[mt][4 * j + 3] * scl};
                *reinterpret_cast<f32x4*>(a.part_acc + row * D + 8 * j + 4 * g2) = o;
            }
        }
    }
}

// LDS of a gather workgroup: the latent operands and four V tiles in the token loop, two publishing slots afterwards
template <int MT>
constexpr size_t gather32_lds()
{
    const size_t main_b = (size_t)MT * 2048 + 4 * 2048;
    const size_t red_b = 2 * ((size_t)MT * 4 * 64 * 16 + 2 * MT * 64 * 4);
    return main_b > red_b ? main_b : red_b;
}

template <int MT>
hipError_t gather32_launch(const MixerArgs& a, hipStream_t st)
{
    auto kern = gather32_kernel<MT>;
    constexpr size_t lds = gather32_lds<MT>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    dim3 grid(a.n_splits * (a.M / (32 * MT)), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a);
    return hipGetLastError();
}

template <int MT>
int gather32_slots()
{
    auto kern = gather32_kernel<MT>;
    constexpr size_t lds = gather32_lds<MT>();
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        (void)hipGetLastError();
    return resident_slots(reinterpret_cast<const void*>(kern), lds);
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

// bf16, D = 32, no key mask; the gather takes latent counts that are multiples of 64 (256, 128 or 64 latents per
// workgroup), the scatter the latent counts its pipeline is unrolled for.
bool mfma32_gather_supported(int dtype, int M, int D, bool masked)
{
    return dtype == 1 && D == 32 && M >= 64 && M % 64 == 0 && !masked;
}

bool mfma32_scatter_supported(int dtype, int M, int D, bool masked)
{
    return dtype == 1 && D == 32 && (M == 64 || M == 128 || M == 256 || M == 512) && !masked;
}

int mfma32_gather_resident_slots(int M)
{
    return M % 256 == 0 ? gather32_slots<8>() : M % 128 == 0 ? gather32_slots<4>() : gather32_slots<2>();
}

hipError_t launch_gather_mfma32(const MixerArgs& a, hipStream_t st)
{
    return a.M % 256 == 0 ? gather32_launch<8>(a, st) : a.M % 128 == 0 ? gather32_launch<4>(a, st) : gather32_launch<2>(a, st);
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
