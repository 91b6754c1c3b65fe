// MFMA (v_mfma_f32_16x16x32_{bf16,f16}) FLARE mixer kernels for gfx950, wave64.
//
// Operand conventions of the 16x16x32 MFMA used throughout (c16 = lane % 16, g = lane / 16):
//   A (16 x 32): lane holds row c16,    k-slots 8g .. 8g+7
//   B (32 x 16): lane holds column c16, k-slots 8g .. 8g+7
//   D (16 x 16): lane holds column c16, rows 4g .. 4g+3 (one per accumulator register)
// A contraction may visit its k index in any order as long as A and B agree, so the
// accumulator of a score tile (rows 4g+r) is fed straight back as the B operand of the
// second product: two score tiles give the 8 k-slots of one lane, no cross-lane traffic.
//
// Scores are produced in log2 units: scale*log2(e) is folded into the latent queries when
// they are converted to MFMA operands, so the steady state per score is exp2 + pack.
// The optimistic pass uses NO softmax shift: fp32 and bf16/f16-as-accumulated share enough exponent
// range that exp2(score) is safe while the scores of a row stay inside (-60, +120); the
// denominators come out of the second product as a row of ones in its A operand and are
// validated after the pass (2^-60 <= l <= 2^120).  What fails validation (and, in the gather,
// a masked range whose real tokens underflow) is recomputed through an exact path with a running maximum.
//
//   gather : z = softmax_n(s q k^T) v   split over N, partial (shift, sum, numerator)
//   scatter: y = softmax_m(s k q^T) z   token parallel, Q and Z^T resident in LDS
#include <mutex>
#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// range of an unshifted softmax denominator that proves no exponential overflowed or lost
// the terms that matter to underflow (2^-60 .. 2^120)
constexpr float kLMin = 8.6736174e-19f, kLMax = 1.329228e36f;

template <typename T> struct Mma;

template <> struct Mma<bf16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static constexpr uint32_t kOnes2 = 0x3f803f80u;   // two bf16 ones
    static __device__ __forceinline__ float dot2(uint32_t x, uint32_t y, float acc)
    {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, y), acc, false);
    }
    static __device__ __forceinline__ float sum2(uint32_t pk, float acc) { return dot2(pk, kOnes2, acc); }
};

template <> struct Mma<f16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static constexpr uint32_t kOnes2 = 0x3c003c00u;   // two f16 ones
    static __device__ __forceinline__ float dot2(uint32_t x, uint32_t y, float acc)
    {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, x), __builtin_bit_cast(f16x2, y), acc, false);
    }
    static __device__ __forceinline__ float sum2(uint32_t pk, float acc) { return dot2(pk, kOnes2, acc); }
};

template <typename T> __device__ __forceinline__ uint16_t elem_bits(float v);
template <> __device__ __forceinline__ uint16_t elem_bits<bf16_t>(float v) { return f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ uint16_t elem_bits<f16_t>(float v)
{
    _Float16 hv = (_Float16)v;
    return __builtin_bit_cast(uint16_t, hv);
}
template <typename T> __device__ __forceinline__ float bits_elem(uint16_t b);
template <> __device__ __forceinline__ float bits_elem<bf16_t>(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
template <> __device__ __forceinline__ float bits_elem<f16_t>(uint16_t b) { return float(__builtin_bit_cast(_Float16, b)); }

__device__ __forceinline__ u32x4 zero4() { return u32x4{0u, 0u, 0u, 0u}; }


// 8 elements (16 bytes) from global memory
__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
// same, for data that is read once: does not displace reusable lines in the caches
__device__ __forceinline__ u32x4 load16_stream(const void* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

// multiply 8 packed elements by f (fp32) and repack
template <typename T> __device__ __forceinline__ u32x4 scale8(u32x4 v, float f)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = bits_elem<T>(uint16_t(v[i] & 0xffffu)) * f;
        const float hi = bits_elem<T>(uint16_t(v[i] >> 16)) * f;
        o[i] = uint32_t(elem_bits<T>(lo)) | (uint32_t(elem_bits<T>(hi)) << 16);
    }
    return o;
}

// 8 packed elements of type T as 8 packed bf16 (identity for bf16)
template <typename T> __device__ __forceinline__ u32x4 to_bf16x8(u32x4 v)
{
    if constexpr (std::is_same<T, bf16_t>::value) return v;
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = Mma<bf16_t>::pack2(bits_elem<T>(uint16_t(v[i] & 0xffffu)), bits_elem<T>(uint16_t(v[i] >> 16)));
    return o;
}

__device__ __forceinline__ float xg_max(float v)  // max over the 4 lane groups of a column
{
    v = max_xor16(v);
    v = max_xor32(v);
    return v;
}
__device__ __forceinline__ float xg_sum(float v)
{
    v = sum_xor16(v);
    v = sum_xor32(v);
    return v;
}

// =====================================================================================
// gather
// =====================================================================================
constexpr int kGTile = 64;            // tokens per barrier step (k-steps of 32)

typedef short s16x4 __attribute__((ext_vector_type(4)));

// LDS transpose read: the 16 lanes of a group each name 8 bytes (4 elements) of a row-major
// tile; lane i of the group receives element i of the four rows named by lane quads 0..3.
__device__ __forceinline__ uint2 lds_read_tr16(const void* lds_addr)
{
    // The pointer reaches the intrinsic through an integer cast, so the compiler may not see that it
    // aliases the ordinary stores that fill the tile: keep it from moving either across the read.
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    asm volatile("" ::: "memory");
    const s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)lds_addr);
    asm volatile("" ::: "memory");
    return __builtin_bit_cast(uint2, r);
}

// One workgroup = 4 waves, 64*CT latents (wave w owns 16*CT of them), one token range.
// K and V tiles of 64 tokens are staged row-major in LDS (double buffered, one barrier per
// tile).  The score product reads K rows as its A operand; the value product needs V^T and
// gets it from the LDS transpose read.  The optimistic pass uses no softmax shift (see the
// scatter kernel); its denominators, produced by a row of ones in the value product, are
// validated at the end and a workgroup that fails repeats its range with a running maximum.
template <typename T, int D, int CT>
__global__ __launch_bounds__(256, 2) void gather_mfma_kernel(MixerArgs a)
{
    constexpr int KD = (D + 31) / 32;   // k-steps over d for the score product
    constexpr int RT = D / 16;          // 16-row tiles of z^T
    constexpr int CH = D / 8;           // 16-byte chunks per row
    constexpr int MB = 64 * CT;
    constexpr int ROWB = D * 2;         // bytes per token row
    constexpr int TILEB = kGTile * ROWB;
    using M_ = Mma<T>;          // score product, in the element type of q and k
    using P_ = Mma<bf16_t>;     // value product: probabilities (and the values they meet) are always bf16

    __shared__ __attribute__((aligned(16))) uint8_t kt[2][TILEB];
    __shared__ __attribute__((aligned(16))) uint8_t vt[2][TILEB];
    __shared__ __attribute__((aligned(16))) uint16_t mt[2][kGTile];   // per token: bf16 1 (real) or 0 (masked / past the range)
    __shared__ int wg_flag[4];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int mblocks = (a.M + MB - 1) / MB;      // M % 64 == 32: the last block's waves 2, 3 own no latent and only help stage
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint8_t* mask = a.mask ? a.mask + (int64_t)b * a.N : nullptr;
    const int m_base = mb * MB + w * 16 * CT;

    // latent operands (B of the score product), log2-scaled
    u32x4 qb[CT][KD];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const int ch = kd * 4 + g;
            qb[ct][kd] = ch < CH && m_base + ct * 16 < a.M
                             ? scale8<T>(load16(q + (int64_t)(m_base + ct * 16 + c16) * a.qs[2] + ch * 8), a.scale_log2)
                             : zero4();
        }
    const u32x4 ones8 = {P_::kOnes2, P_::kOnes2, P_::kOnes2, P_::kOnes2};

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);

    // staging: 16-byte chunk c of a tile = (token c / CH, chunk c % CH); rows beyond n_end are
    // clamped to the last valid row (their probabilities are forced to 0 below)
    constexpr int TCH = kGTile * CH;
    constexpr int CPT = (TCH + 255) / 256;
    // K chunks are XOR-swizzled by (token / 4) so that the 16 rows an A-operand read touches
    // fall into distinct banks; V rows swap their 32-byte halves on odd (token / 4) for the
    // transpose read
    auto k_slot = [](int tok, int ch) { return tok * ROWB + ((ch ^ ((tok >> 2) & (CH - 1))) << 4); };
    auto v_slot = [](int tok, int ch) { return tok * ROWB + ((CH >= 4 ? (ch ^ (((tok >> 2) & 1) << 1)) : ch) << 4); };

    // two register sets: tiles are fetched two iterations before they are consumed.  With a key mask (MASKED) a
    // token that is padded or lies past the range keeps a (finite) K row but gets a zero V row and a zero in the
    // tile's row of "ones": whatever its probability, it adds nothing to the numerators or the denominators.
    u32x4 kr[2][CPT], vr[2][CPT];
    // the token's mask byte as loaded and "inside the range": combined only where the tile is stored -- a flag computed
    // from the byte at the load would wait for it there, and with it, in order, for the K and V rows requested just before
    uint32_t mbyte[2][CPT];
    bool inr[2][CPT];
    auto load_tile = [&](auto set_tag, int n0, auto masked_tag) {
        constexpr int S = decltype(set_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * 256;
            if (TCH % 256 == 0 || c < TCH) {
                const int nn = n0 + c / CH, n = max(min(nn, n_end - 1), 0), ch = c % CH;
                kr[S][i] = load16_stream(k + (int64_t)n * a.ks[2] + ch * 8);
                vr[S][i] = load16_stream(v + (int64_t)n * a.vs[2] + ch * 8);
                if constexpr (MASKED) {
                    mbyte[S][i] = mask[n];
                    inr[S][i] = nn < n_end;
                }
            }
        }
    };
    auto store_tile = [&](auto set_tag, auto masked_tag) {   // register set S always feeds LDS buffer S
        constexpr int S = decltype(set_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * 256;
            if (TCH % 256 == 0 || c < TCH) {
                const int tok = c / CH, ch = c % CH;
                *reinterpret_cast<u32x4*>(&kt[S][k_slot(tok, ch)]) = kr[S][i];
                if constexpr (MASKED) {
                    const bool live = inr[S][i] && mbyte[S][i] != 0;
                    *reinterpret_cast<u32x4*>(&vt[S][v_slot(tok, ch)]) = live ? to_bf16x8<T>(vr[S][i]) : zero4();
                    if (ch == 0) mt[S][tok] = live ? uint16_t(P_::kOnes2 & 0xffffu) : uint16_t(0);
                } else {
                    *reinterpret_cast<u32x4*>(&vt[S][v_slot(tok, ch)]) = to_bf16x8<T>(vr[S][i]);
                }
            }
        }
    };
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;

    float shift[CT];
    f32x4 zacc[RT][CT], lacc[CT];
    // With attention dropout the optimistic pass is skipped: the keep mask is applied element by element in the exact pass.
    const bool drop = a.drop_thr != 0;

    // one pass over the token range; EXACT keeps a running maximum per latent
    // MASKED: the problem has a key mask (decided once per launch, so the unmasked instance carries none of it)
    auto run = [&](auto exact_tag, auto masked_tag) {
        constexpr bool EXACT = decltype(exact_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            shift[ct] = EXACT ? kNegBig : 0.f;
            lacc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) zacc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        // tile i lives in LDS buffer i & 1; it is written there one iteration before its use from
        // the register set of the same parity, which was loaded two iterations before
        auto process = [&](int n0, int buf) {
            const bool ragged = MASKED || (n0 + kGTile > n_end);
            auto tile = [&](auto ragged_tag) {
                constexpr bool RAGGED = decltype(ragged_tag)::value;
                // the optimistic pass of a masked problem runs every tile through the pipelined loop with the tile's
                // live-token row as its row of "ones", read once per tile: lane (c16, g) meets tokens 4g..4g+3 of
                // both 16-token sub-tiles of a k-step.  Without a mask only the one ragged tile at the end of a range
                // leaves the pipelined loop (element-wise selects below).
                constexpr bool PIPELINED = !EXACT && (MASKED || !RAGGED);
                u32x4 ones_t[kGTile / 32];
                if constexpr (PIPELINED && MASKED) {
#pragma unroll
                    for (int ks = 0; ks < kGTile / 32; ++ks) {
                        const uint2 lo = *reinterpret_cast<const uint2*>(&mt[buf][ks * 32 + 4 * g]);
                        const uint2 hi = *reinterpret_cast<const uint2*>(&mt[buf][ks * 32 + 16 + 4 * g]);
                        ones_t[ks] = u32x4{lo.x, lo.y, hi.x, hi.y};
                    }
                }
#pragma unroll
                for (int ks = 0; ks < kGTile / 32; ++ks) {
                    // operands: two 16-token K sub-tiles (A of the score product), V^T (A of the value product)
                    u32x4 ka0[KD], ka1[KD], va[RT];
    #pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        const int ch = kd * 4 + g;
                        const int t0 = ks * 32 + c16, t1 = t0 + 16;
                        ka0[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&kt[buf][k_slot(t0, ch)]) : zero4();
                        ka1[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&kt[buf][k_slot(t1, ch)]) : zero4();
                    }
    #pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        // lane (c16, g): rows 4g + (c16 >> 2) of each sub-tile, 8 bytes at d = 16 rt + 4 (c16 & 3)
                        const int r0 = ks * 32 + 4 * g + (c16 >> 2), r1 = r0 + 16;
                        const int ch = 2 * rt + ((c16 & 3) >> 1), sub = (c16 & 1) << 3;
                        const uint2 lo = lds_read_tr16(&vt[buf][v_slot(r0, ch) + sub]);
                        const uint2 hi = lds_read_tr16(&vt[buf][v_slot(r1, ch) + sub]);
                        va[rt] = u32x4{lo.x, lo.y, hi.x, hi.y};
                    }
                    if constexpr (PIPELINED) {
                        // steady state: latent tiles software pipelined (scores of tile ct+1 issued before
                        // the exponentials of tile ct, value product of tile ct-1 after them)
                        u32x4 ones_a = ones8;
                        if constexpr (MASKED) ones_a = ones_t[ks];
                        auto sc2 = [&](int ct, f32x4& s0, f32x4& s1) {
                            s0 = f32x4{0.f, 0.f, 0.f, 0.f};
                            s1 = s0;
    #pragma unroll
                            for (int kd = 0; kd < KD; ++kd) {
                                s0 = M_::mma(ka0[kd], qb[ct][kd], s0);
                                s1 = M_::mma(ka1[kd], qb[ct][kd], s1);
                            }
                        };
                        auto pv = [&](int ct, u32x4 pb) {
    #pragma unroll
                            for (int rt = 0; rt < RT; ++rt) zacc[rt][ct] = P_::mma(va[rt], pb, zacc[rt][ct]);
                            lacc[ct] = P_::mma(ones_a, pb, lacc[ct]);   // row of ones: the softmax denominator
                        };
                        f32x4 s0, s1;
                        sc2(0, s0, s1);
                        u32x4 pbp = zero4();
    #pragma unroll
                        for (int ct = 0; ct < CT; ++ct) {
                            // waves that are issuing matrix products go first: the other waves' exponentials fill in behind them
                            __builtin_amdgcn_s_setprio(1);
                            f32x4 n0 = s0, n1 = s1;
                            if (ct + 1 < CT) sc2(ct + 1, n0, n1);
                            if (ct > 0) pv(ct - 1, pbp);
                            __builtin_amdgcn_sched_barrier(0);     // matrix products first: the exponentials run under them
                            __builtin_amdgcn_s_setprio(0);
                            __builtin_amdgcn_sched_barrier(0);
                            const u32x4 pb = {P_::pack2(fast_exp2(s0[0]), fast_exp2(s0[1])),
                                              P_::pack2(fast_exp2(s0[2]), fast_exp2(s0[3])),
                                              P_::pack2(fast_exp2(s1[0]), fast_exp2(s1[1])),
                                              P_::pack2(fast_exp2(s1[2]), fast_exp2(s1[3]))};
                            s0 = n0;
                            s1 = n1;
                            pbp = pb;
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        pv(CT - 1, pbp);
                    } else
    #pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    #pragma unroll
                        for (int kd = 0; kd < KD; ++kd) {
                            s0 = M_::mma(ka0[kd], qb[ct][kd], s0);
                            s1 = M_::mma(ka1[kd], qb[ct][kd], s1);
                        }
                        float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
                        bool ok[8];
                        if (EXACT || RAGGED) {
    #pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const int n = n0 + ks * 32 + (e >> 2) * 16 + 4 * g + (e & 3);
                                ok[e] = !RAGGED || (n < n_end && (mask == nullptr || mask[n] != 0));
                            }
                        }
                        if (EXACT) {
                            float mx = kNegBig;
    #pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (ok[e]) mx = fmaxf(mx, sc[e]);
                            mx = xg_max(mx);
                            const float nc = fmaxf(shift[ct], mx);
                            const float al = fast_exp2(shift[ct] - nc);
    #pragma unroll
                            for (int rt = 0; rt < RT; ++rt) zacc[rt][ct] *= al;
                            lacc[ct] *= al;
                            shift[ct] = nc;
    #pragma unroll
                            for (int e = 0; e < 8; ++e) sc[e] -= nc;
                        }
                        float p[8];
    #pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            p[e] = fast_exp2(sc[e]);
                            if (EXACT || RAGGED) p[e] = ok[e] ? p[e] : 0.f;
                        }
                        const u32x4 pb = {P_::pack2(p[0], p[1]), P_::pack2(p[2], p[3]),
                                          P_::pack2(p[4], p[5]), P_::pack2(p[6], p[7])};
                        u32x4 pbv = pb;
                        if (EXACT && drop) {
                            // attention dropout: the denominator keeps every weight, the value product meets the kept
                            // ones (their common factor 1 / (1 - p) is applied to the partial at the end)
                            const uint32_t m = (uint32_t)(m_base + ct * 16 + c16), bh = (uint32_t)(b * a.H + h);
    #pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const uint32_t n = (uint32_t)(n0 + ks * 32 + (e >> 2) * 16 + 4 * g + (e & 3));
                                p[e] = dropout_hash24(a.seed_lo, a.seed_hi, 0u, bh, m, n) >= a.drop_thr ? p[e] : 0.f;
                            }
                            pbv = u32x4{P_::pack2(p[0], p[1]), P_::pack2(p[2], p[3]), P_::pack2(p[4], p[5]), P_::pack2(p[6], p[7])};
                        }
    #pragma unroll
                        for (int rt = 0; rt < RT; ++rt) zacc[rt][ct] = P_::mma(va[rt], pbv, zacc[rt][ct]);
                        lacc[ct] = P_::mma(ones8, pb, lacc[ct]);   // row of ones: the softmax denominator
                    }
                }
    };
            if (ragged) tile(std::true_type{});
            else        tile(std::false_type{});
        };
        // Loads and LDS stores of the staging are unconditional (rows past the range repeat its last row, a tile past
        // it is staged and never read) and the loop over pairs of tiles has its one exit at the bottom: with a branch
        // around a load, or a way from the middle of the pair back to the loop's head, the compiler cannot count the
        // loads in flight and waits for all of them at every tile, the ones requested an iteration ago included.
        auto iter = [&](int n0, auto par) {
            constexpr int P = decltype(par)::value;
            using Other = std::integral_constant<int, 1 - P>;
            __syncthreads();
            store_tile(Other{}, masked_tag);
            load_tile(Other{}, n0 + 3 * kGTile, masked_tag);
            process(n0, P);
        };
        const int tiles = n_begin < n_end ? (n_end - n_begin + kGTile - 1) / kGTile : 0;
        if (tiles > 0) {
            load_tile(Set0{}, n_begin, masked_tag);
            load_tile(Set1{}, n_begin + kGTile, masked_tag);
            store_tile(Set0{}, masked_tag);
            load_tile(Set0{}, n_begin + 2 * kGTile, masked_tag);
        }
        int n0 = n_begin;
        for (int i = 0; i < tiles / 2; ++i, n0 += 2 * kGTile) {
            iter(n0, Set0{});
            iter(n0 + kGTile, Set1{});
        }
        if (tiles & 1) iter(n0, Set0{});
    };

    // validate: every denominator of this wave inside the safe range, numerators finite.  With a key mask a
    // range without a single real token legitimately gives l = 0: the lower bound applies only when the
    // range holds one (counted here; the mask and the range are uniform over the workgroup).
    bool exact = true;
    if (!drop) {
        int has_valid = n_begin < n_end;
        if (mask != nullptr) {
            run(std::false_type{}, std::true_type{});
            int any = 0;
            for (int n = n_begin + tid; n < n_end; n += 256) any |= mask[n];
            has_valid = __syncthreads_or(any);
        } else {
            run(std::false_type{}, std::false_type{});
        }
        bool bad = false;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const float l = lacc[ct][0];
            bad = bad || !(l <= kLMax) || (has_valid && !(l >= kLMin));
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int r = 0; r < 4; ++r) bad = bad || !(fabsf(zacc[rt][ct][r]) <= 3.0e38f);
        }
        const int anybad = __any(bad);
        __syncthreads();
        if (lane == 0) wg_flag[w] = anybad;
        __syncthreads();
        exact = (wg_flag[0] | wg_flag[1] | wg_flag[2] | wg_flag[3]) != 0;
    }
    if (exact) {
        asm volatile("; exact pass" ::: "memory");
        if (mask != nullptr) run(std::true_type{}, std::true_type{});
        else                 run(std::true_type{}, std::false_type{});
    }

    // partial for this split: shift (log2 units), sum, numerator, renormalised so that the
    // sum has exponent 0 (keeps the merge free of overflow whatever the pass left behind)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const float l = lacc[ct][0];
        int e = 0;
        if (l > 0.f) (void)frexpf(l, &e);
        const float sc = l > 0.f ? ldexpf(1.f, -e) : 0.f;
        const int m = m_base + ct * 16 + c16;
        if (m >= a.M) continue;
        const int64_t row = (((int64_t)b * a.H + h) * a.n_parts + split) * a.M + m;
        if (g == 0) {
            a.part_m[row] = l > 0.f ? shift[ct] + (float)e : kNegBig;
            a.part_l[row] = l * sc;
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
            *reinterpret_cast<f32x4*>(a.part_acc + row * D + rt * 16 + 4 * g) = zacc[rt][ct] * (drop ? sc * a.drop_rs : sc);
    }
}

// =====================================================================================
// scatter
// =====================================================================================
// 16-token column tiles per wave iteration: 4, and 2 at D = 64, where the accumulators and K operands of 4
// tiles do not fit the register file (84 registers spilled, and twice the time per score)
constexpr int scatter_tiles(int D) { return D <= 32 ? 4 : 2; }

// One workgroup = 4 independent waves sharing Q and Z^T operands in LDS; wave w walks the
// workgroup's token range in steps of 64 tokens.  No barrier after the set-up.
// KSC = M / 32 fixed at compile time (the latent loop is then fully unrolled, operands renamed
// instead of copied, accumulators started from a literal zero) or 0 for any M at run time.
// Inside a latent step the 4 token tiles are software pipelined: the scores of tile t+1 are
// issued before the exponentials of tile t, and the value product of tile t-1 after them, so
// that no instruction waits on the matrix-core result just issued.
template <typename T, int D, int KSC>
__global__ __launch_bounds__(256, 2) void scatter_mfma_kernel(MixerArgs a, int tokens_per_wg)
{
    constexpr int KD = (D + 31) / 32;
    constexpr int RT = D / 16;
    constexpr int CH = D / 8;
    constexpr int kSTW = scatter_tiles(D), kSTokWave = 16 * kSTW;
    using M_ = Mma<T>;          // score product, in the element type of q and k
    using P_ = Mma<bf16_t>;     // value product: probabilities (and the values they meet) are always bf16

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // qa[mt][ch][c16]  : 16 bytes each, latent m = 16 mt + c16, d = 8 ch .. 8 ch + 7
    // zt[ks][rt][lane] : 16 bytes each, row d = (D/4) (c16/4) + 4 rt + c16 % 4,
    //                    slots e<4 -> m = 32 ks + 4 g + e, e>=4 -> m = 32 ks + 16 + 4 g + e - 4
    u32x4* qa = reinterpret_cast<u32x4*>(smem);
    u32x4* zt = qa + (size_t)a.M * CH;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const int M = KSC ? 32 * KSC : a.M, KS = M / 32;

    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    uint16_t* y = (uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    const float* z = a.z + ((int64_t)b * a.H + h) * M * D;
    const uint8_t* mask = a.mask ? a.mask + (int64_t)b * a.N : nullptr;

    for (int idx = tid; idx < M * CH; idx += 256) {
        const int m = idx / CH, ch = idx % CH;
        qa[((m >> 4) * CH + ch) * 16 + (m & 15)] =
            scale8<T>(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2);
    }
    for (int idx = tid; idx < KS * RT * 64; idx += 256) {
        const int ln = idx & 63, rt = (idx >> 6) % RT, ks = idx / (64 * RT);
        const int cc = ln & 15, gg = ln >> 4;
        const int d = (D / 4) * (cc >> 2) + 4 * rt + (cc & 3);
        u32x4 o;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            const int e = 2 * e2;
            const int m0 = 32 * ks + (e >> 2) * 16 + 4 * gg + (e & 3);
            o[e2] = uint32_t(elem_bits<bf16_t>(z[(int64_t)m0 * D + d])) |
                    (uint32_t(elem_bits<bf16_t>(z[(int64_t)(m0 + 1) * D + d])) << 16);
        }
        zt[idx] = o;
    }
    __syncthreads();

    const int wg_n0 = blockIdx.x * tokens_per_wg;
    const int wg_n1 = min(a.N, wg_n0 + tokens_per_wg);
    const u32x4 ones8 = {P_::kOnes2, P_::kOnes2, P_::kOnes2, P_::kOnes2};
    const f32x4 zf = {0.f, 0.f, 0.f, 0.f};

    // (the tokens' mask bytes travel with their K rows: loaded where a tile's rows are stored, the byte would be waited for
    // on the spot, and with it, in order, the K rows of the next tile requested before)
    auto load_k = [&](int t0, u32x4 (&dst)[kSTW][KD], uint32_t (&mdst)[kSTW]) {
#pragma unroll
        for (int tw = 0; tw < kSTW; ++tw) {
            const int n = t0 + tw * 16 + c16;
            mdst[tw] = mask != nullptr ? (uint32_t)mask[n < wg_n1 ? n : wg_n1 - 1] : 1u;
        }
        if (CH == 4 * KD && t0 + kSTokWave <= wg_n1) {      // wave-uniform: whole tile in range, no per-lane tests
            const uint16_t* kr = k + (int64_t)(t0 + c16) * a.ks[2] + g * 8;
#pragma unroll
            for (int tw = 0; tw < kSTW; ++tw)
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) dst[tw][kd] = load16_stream(kr + (int64_t)tw * 16 * a.ks[2] + kd * 32);
            return;
        }
#pragma unroll
        for (int tw = 0; tw < kSTW; ++tw)
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                const int n = t0 + tw * 16 + c16, ch = kd * 4 + g;
                dst[tw][kd] = (n < wg_n1 && ch < CH) ? load16_stream(k + (int64_t)n * a.ks[2] + ch * 8) : zero4();
            }
    };
    auto load_ops = [&](int ks, u32x4 (&o0)[KD], u32x4 (&o1)[KD], u32x4 (&oz)[RT]) {
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const int ch = kd * 4 + g;
            o0[kd] = ch < CH ? qa[((2 * ks) * CH + ch) * 16 + c16] : zero4();
            o1[kd] = ch < CH ? qa[((2 * ks + 1) * CH + ch) * 16 + c16] : zero4();
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) oz[rt] = zt[(ks * RT + rt) * 64 + lane];
    };
    auto scores = [&](const u32x4 (&o)[KD], const u32x4 (&kk)[KD]) {
        f32x4 s = zf;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) s = M_::mma(o[kd], kk[kd], s);
        return s;
    };

    // one 64-token tile of this wave: kb = its K rows as B operands
    auto tile64 = [&](const u32x4 (&kb)[kSTW][KD], const uint32_t (&mb)[kSTW], int t0) {
        f32x4 yacc[kSTW][RT];
        float lrow[kSTW];       // softmax denominators, complete for the lane's token
        float lshift[kSTW];     // log2 shift the denominators are relative to (0 in the optimistic pass)
        bool redo = false;
#pragma unroll
        for (int tw = 0; tw < kSTW; ++tw) lshift[tw] = 0.f;
        const bool drop = a.drop_thr != 0;      // attention dropout: straight to the element-wise exact path
        if (drop) {
            redo = true;
        } else {
            // Optimistic pass: no softmax shift at all.  fp32 and bf16 share an 8-bit exponent, so
            // exp2(score) is exact enough whenever the scores of a token stay inside (-60, 120);
            // that is validated afterwards on the denominators, and only a token tile that
            // fails goes through the exact (running maximum) path below.
            f32x4 yl[kSTW];
            u32x4 q0[KD], q1[KD], za[RT], q0n[KD], q1n[KD], zan[RT];
            // one latent step (32 latents) for the wave's 4 column tiles, pipelined over the tiles
            auto step = [&](bool first) {
                auto pv = [&](int tw, u32x4 pb) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) yacc[tw][rt] = P_::mma(za[rt], pb, first ? zf : yacc[tw][rt]);
                    yl[tw] = P_::mma(ones8, pb, first ? zf : yl[tw]);   // row of ones: the softmax denominator
                };
                f32x4 s0 = scores(q0, kb[0]), s1 = scores(q1, kb[0]);
                u32x4 pbp = zero4();
#pragma unroll
                for (int tw = 0; tw < kSTW; ++tw) {
                    __builtin_amdgcn_s_setprio(1);      // as in the gather: matrix-product issue takes precedence
                    f32x4 n0 = zf, n1 = zf;
                    if (tw + 1 < kSTW) {
                        n0 = scores(q0, kb[tw + 1]);
                        n1 = scores(q1, kb[tw + 1]);
                    }
                    if (tw > 0) pv(tw - 1, pbp);
                    __builtin_amdgcn_sched_barrier(0);     // matrix products first: the exponentials run under them
                    __builtin_amdgcn_s_setprio(0);
                    __builtin_amdgcn_sched_barrier(0);
                    const u32x4 pb = {P_::pack2(fast_exp2(s0[0]), fast_exp2(s0[1])),
                                      P_::pack2(fast_exp2(s0[2]), fast_exp2(s0[3])),
                                      P_::pack2(fast_exp2(s1[0]), fast_exp2(s1[1])),
                                      P_::pack2(fast_exp2(s1[2]), fast_exp2(s1[3]))};
                    s0 = n0;
                    s1 = n1;
                    pbp = pb;
                    __builtin_amdgcn_sched_barrier(0);
                }
                pv(kSTW - 1, pbp);
            };
            auto advance = [&](int ks) {   // operands of step ks become current, those of ks + 1 are fetched
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) {
                    q0[kd] = q0n[kd];
                    q1[kd] = q1n[kd];
                }
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) za[rt] = zan[rt];
                if (ks + 1 < KS) load_ops(ks + 1, q0n, q1n, zan);
            };
            load_ops(0, q0, q1, za);
            if (KS > 1) load_ops(1, q0n, q1n, zan);
            step(true);
            if constexpr (KSC > 0) {
#pragma unroll
                for (int ks = 1; ks < KSC; ++ks) {
                    advance(ks);
                    step(false);
                }
            } else {
#pragma unroll 1
                for (int ks = 1; ks < KS; ++ks) {
                    advance(ks);
                    step(false);
                }
            }
#pragma unroll
            for (int tw = 0; tw < kSTW; ++tw) {
                lrow[tw] = yl[tw][0];
                redo = redo || !(lrow[tw] >= kLMin && lrow[tw] <= kLMax);
            }
        }
        if (__builtin_expect(__any(redo), 0)) {
            // exact path: online maximum with rescaling
            asm volatile("; exact path" ::: "memory");
            float shift[kSTW], lsum[kSTW];
#pragma unroll
            for (int tw = 0; tw < kSTW; ++tw) {
                shift[tw] = kNegBig;
                lsum[tw] = 0.f;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) yacc[tw][rt] = zf;
            }
#pragma unroll 1
            for (int ks = 0; ks < KS; ++ks) {
                u32x4 q0[KD], q1[KD], za[RT];
                load_ops(ks, q0, q1, za);
#pragma unroll
                for (int tw = 0; tw < kSTW; ++tw) {
                    const f32x4 s0 = scores(q0, kb[tw]), s1 = scores(q1, kb[tw]);
                    float mx = fmaxf(fmaxf(fmaxf(s0[0], s0[1]), fmaxf(s0[2], s0[3])),
                                     fmaxf(fmaxf(s1[0], s1[1]), fmaxf(s1[2], s1[3])));
                    mx = xg_max(mx);
                    const float nc = fmaxf(shift[tw], mx);
                    const float al = fast_exp2(shift[tw] - nc);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) yacc[tw][rt] *= al;
                    lsum[tw] *= al;
                    shift[tw] = nc;
                    const u32x4 pb = {P_::pack2(fast_exp2(s0[0] - nc), fast_exp2(s0[1] - nc)),
                                      P_::pack2(fast_exp2(s0[2] - nc), fast_exp2(s0[3] - nc)),
                                      P_::pack2(fast_exp2(s1[0] - nc), fast_exp2(s1[1] - nc)),
                                      P_::pack2(fast_exp2(s1[2] - nc), fast_exp2(s1[3] - nc))};
                    float t = P_::sum2(pb[0], 0.f);
                    t = P_::sum2(pb[1], t);
                    t = P_::sum2(pb[2], t);
                    t = P_::sum2(pb[3], t);
                    lsum[tw] += t;
                    u32x4 pbv = pb;
                    if (drop) {     // the denominator keeps every weight, the value product meets the kept ones
                        const uint32_t n = (uint32_t)min(t0 + tw * 16 + c16, a.N - 1), bh = (uint32_t)(b * a.H + h);
                        float pd[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const uint32_t m = (uint32_t)(32 * ks + (e >> 2) * 16 + 4 * g + (e & 3));
                            const float pe = fast_exp2((e < 4 ? s0[e & 3] : s1[e & 3]) - nc);
                            pd[e] = dropout_hash24(a.seed_lo, a.seed_hi, 1u, bh, m, n) >= a.drop_thr ? pe : 0.f;
                        }
                        pbv = u32x4{P_::pack2(pd[0], pd[1]), P_::pack2(pd[2], pd[3]), P_::pack2(pd[4], pd[5]), P_::pack2(pd[6], pd[7])};
                    }
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) yacc[tw][rt] = P_::mma(za[rt], pbv, yacc[tw][rt]);
                }
            }
#pragma unroll
            for (int tw = 0; tw < kSTW; ++tw) {
                lrow[tw] = xg_sum(lsum[tw]);
                lshift[tw] = shift[tw];
            }
        }

        // normalise and store: lane (token c16, group g) owns d = (D/4) g .. (D/4) g + D/4 - 1
        const bool full = t0 + kSTokWave <= wg_n1 && mask == nullptr;   // wave-uniform: no per-row tests
        uint16_t* yr0 = y + (int64_t)(t0 + c16) * a.ys[2] + (D / 4) * g;
        auto emit = [&](auto full_c) {
            constexpr bool FULL = decltype(full_c)::value;
#pragma unroll
            for (int tw = 0; tw < kSTW; ++tw) {
                const int n = t0 + tw * 16 + c16;
                const bool in = FULL || n < wg_n1;
                const bool on = FULL || (in && mb[tw] != 0);
                const float inv = on ? __builtin_amdgcn_rcpf(lrow[tw]) * (drop ? a.drop_rs : 1.f) : 0.f;
                if (in) {
                    uint16_t* yr = yr0 + (int64_t)tw * 16 * a.ys[2];
                    uint32_t o[2 * RT];
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        f32x4 yv = yacc[tw][rt] * inv;
                        if (!FULL && !on) yv = f32x4{0.f, 0.f, 0.f, 0.f};      // a padded row is 0 whatever its key row held
                        o[2 * rt] = M_::pack2(yv[0], yv[1]);
                        o[2 * rt + 1] = M_::pack2(yv[2], yv[3]);
                    }
                    if constexpr (RT == 1) {
                        *reinterpret_cast<uint2*>(yr) = make_uint2(o[0], o[1]);
                    } else {
#pragma unroll
                        for (int i = 0; i < RT / 2; ++i) {
                            const u32x4 ov = {o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
                            __builtin_nontemporal_store(ov, reinterpret_cast<u32x4*>(yr + 8 * i));   // written once, never re-read here
                        }
                    }
                }
            }
            if (a.lse_tok) {        // log-sum-exp of the token's scores, for the backward pass
                float* lo = a.lse_tok + ((int64_t)b * a.H + h) * a.N + t0 + c16;
#pragma unroll
                for (int tw = 0; tw < kSTW; ++tw)
                    if (g == 0 && (FULL || t0 + tw * 16 + c16 < wg_n1)) lo[tw * 16] = (lshift[tw] + __log2f(lrow[tw])) * kLn2;
            }
        };
        if (full) emit(std::true_type{}); else emit(std::false_type{});
    };

    // two K register sets alternate, each fetched one tile before its use
    u32x4 ka[kSTW][KD], kc[kSTW][KD];
    uint32_t ma[kSTW], mc[kSTW];
    constexpr int kStride = 4 * kSTokWave;
    int t0 = wg_n0 + w * kSTokWave;
    if (t0 < wg_n1) load_k(t0, ka, ma);
    for (; t0 < wg_n1; t0 += 2 * kStride) {
        if (t0 + kStride < wg_n1) load_k(t0 + kStride, kc, mc);
        tile64(ka, ma, t0);
        if (t0 + kStride < wg_n1) {
            if (t0 + 2 * kStride < wg_n1) load_k(t0 + 2 * kStride, ka, ma);
            tile64(kc, mc, t0 + kStride);
        }
    }
}

constexpr size_t kScatterLdsMax = 150 * 1024;

template <typename T, int D>
const void* gather_kernel_ptr(int M)
{
    if constexpr (D <= 32) {
        if (M % 256 == 0) return reinterpret_cast<const void*>(gather_mfma_kernel<T, D, 4>);
    }
    if (M % 128 == 0) return reinterpret_cast<const void*>(gather_mfma_kernel<T, D, 2>);
    return reinterpret_cast<const void*>(gather_mfma_kernel<T, D, 1>);
}

template <typename T>
const void* gather_kernel_ptr_d(int M, int D)
{
    switch (D) {
        case 16: return gather_kernel_ptr<T, 16>(M);
        case 32: return gather_kernel_ptr<T, 32>(M);
        default: return gather_kernel_ptr<T, 64>(M);
    }
}

template <typename T, int D>
hipError_t gather_launch_ct(const MixerArgs& a, hipStream_t st)
{
    // 64 latents per wave only up to D = 32: at D = 64 that instance spills 445 registers
    const int MB = (a.M % 256 == 0 && D <= 32) ? 256 : (a.M % 128 == 0) ? 128 : 64;
    dim3 grid(a.n_splits * ((a.M + MB - 1) / MB), a.H, a.B);
    if constexpr (D <= 32) {
        if (MB == 256) {
            hipLaunchKernelGGL((gather_mfma_kernel<T, D, 4>), grid, dim3(256), 0, st, a);
            return hipGetLastError();
        }
    }
    if (MB == 128) hipLaunchKernelGGL((gather_mfma_kernel<T, D, 2>), grid, dim3(256), 0, st, a);
    else           hipLaunchKernelGGL((gather_mfma_kernel<T, D, 1>), grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

template <typename T>
hipError_t gather_launch_d(const MixerArgs& a, hipStream_t st)
{
    switch (a.D) {
        case 16: return gather_launch_ct<T, 16>(a, st);
        case 32: return gather_launch_ct<T, 32>(a, st);
        case 64: return gather_launch_ct<T, 64>(a, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, int D>
hipError_t scatter_launch(const MixerArgs& a, hipStream_t st)
{
    const size_t lds = (size_t)a.M * D * 2 * 2;
    // the latent loop is unrolled at compile time for the usual latent counts at D <= 32
    auto kern = scatter_mfma_kernel<T, D, 0>;
    if constexpr (D <= 32) {
        switch (a.M) {
            case 64:  kern = scatter_mfma_kernel<T, D, 2>; break;
            case 128: kern = scatter_mfma_kernel<T, D, 4>; break;
            case 256: kern = scatter_mfma_kernel<T, D, 8>; break;
            case 512: kern = scatter_mfma_kernel<T, D, 16>; break;
            default: break;
        }
    }
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    // tokens per workgroup (multiple of 256): one full round of resident workgroups when the
    // problem is large enough, so that every CU finishes at the same time
    const int slots = resident_slots(reinterpret_cast<const void*>(kern), lds);
    const int64_t per_bh = (slots + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H);   // workgroups per (b,h)
    int64_t tpw = (a.N + per_bh - 1) / per_bh;
    tpw = ((tpw + 255) / 256) * 256;
    if (tpw < 256) tpw = 256;       // one 64-token pass per wave: a launch this small is bound by latency, not by the operand set-up
    dim3 grid((unsigned)((a.N + tpw - 1) / tpw), a.H, a.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a, (int)tpw);
    return hipGetLastError();
}

template <typename T>
hipError_t scatter_launch_d(const MixerArgs& a, hipStream_t st)
{
    switch (a.D) {
        case 16: return scatter_launch<T, 16>(a, st);
        case 32: return scatter_launch<T, 32>(a, st);
        case 64: return scatter_launch<T, 64>(a, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// Workgroups of `kern` the current device holds at once (CUs x occupancy).  Grids are sized
// to a whole multiple of this so that no partially filled last round is left over.
// Falls back to 2 per CU on 256 CUs when no device can be queried (host-only planning).
int resident_slots(const void* kern, size_t dyn_lds, int block_threads)
{
    struct Entry { const void* k; size_t lds; int dev; int slots; };
    static Entry cache[64];
    static int ncache = 0;
    static std::mutex mu;     // the cache is the only mutable state of the library: guard it
    std::lock_guard<std::mutex> lock(mu);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return 512; }
    for (int i = 0; i < ncache; ++i)
        if (cache[i].k == kern && cache[i].lds == dyn_lds && cache[i].dev == dev) return cache[i].slots;
    int occ = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kern, block_threads, dyn_lds) != hipSuccess || occ < 1) {
        (void)hipGetLastError();
        return 512;
    }
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
        (void)hipGetLastError();
        return 512;
    }
    const int slots = occ * cus;
    if (ncache < 64) cache[ncache++] = Entry{kern, dyn_lds, dev, slots};
    return slots;
}

// Compute units of the current device (256 when no device can be queried: host-only planning).
int device_cus()
{
    static int cached[64];
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return 256; }
    if (dev >= 0 && dev < 64 && cached[dev] > 0) return cached[dev];
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
        (void)hipGetLastError();
        return 256;
    }
    if (dev >= 0 && dev < 64) cached[dev] = cus;
    return cus;
}

bool mfma_mixer_supported(int dtype, int M, int D)
{
    if (dtype != 1 && dtype != 2) return false;
    if (D != 16 && D != 32 && D != 64) return false;
    if (M < 32 || M % 32 != 0) return false;      // the scatter walks the latents 32 at a time, the gather pads its last block
    if ((size_t)M * D * 4 > kScatterLdsMax) return false;
    return true;
}

// Token granularity of a gather split: the 64-token tile of the 16x16x32 kernel, or one 32-token pass of each of
// the four waves of the 32x32x16 kernel.  The plan depends on the descriptor only; a launch that turns out to carry a
// key mask runs the 16x16x32 kernel on the same split, which it takes as well.
int mfma_gather_tokens_per_iter(int dtype, int M, int D, bool allow32)
{
    return allow32 && mfma32_gather_supported(dtype, M, D, false) ? 128 : kGTile;
}

int mfma_gather_resident_slots(int dtype, int M, int D, bool allow32)
{
    if (allow32 && mfma32_gather_supported(dtype, M, D, false)) return mfma32_gather_resident_slots(M);
    const void* k = dtype == 1 ? gather_kernel_ptr_d<bf16_t>(M, D) : gather_kernel_ptr_d<f16_t>(M, D);
    return resident_slots(k, 0);
}

hipError_t launch_gather_mfma(const MixerArgs& a, int dtype, hipStream_t st)
{
    if (!a.no_mfma32 && mfma32_gather_supported(dtype, a.M, a.D, a.mask != nullptr)) return launch_gather_mfma32(a, st);
    return dtype == 1 ? gather_launch_d<bf16_t>(a, st) : gather_launch_d<f16_t>(a, st);
}

hipError_t launch_scatter_mfma(const MixerArgs& a, int dtype, hipStream_t st)
{
    if (!a.no_mfma32 && mfma32_scatter_supported(dtype, a.M, a.D, a.mask != nullptr)) return launch_scatter_mfma32(a, st);
    return dtype == 1 ? scatter_launch_d<bf16_t>(a, st) : scatter_launch_d<f16_t>(a, st);
}

}  // namespace flare
