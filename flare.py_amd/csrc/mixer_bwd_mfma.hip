// Backward of the FLARE mixer on the matrix cores (bf16 / f16, no key mask).
//
// Forward (README.md:39-52 of the reference):  S[m,n] = s <q_m,k_n>,  z_m = sum_n A[m,n] v_n with
// A = softmax over n,  y_n = sum_m Bt[n,m] z_m with Bt = softmax over m.  With L_m, rho_n the two
// log-sum-exps saved by the forward:  A[m,n] = exp(S - L_m) <= 1,  Bt[n,m] = exp(S - rho_n) <= 1.
// Given dy:
//   delta_n = <dy_n, y_n>                          (bwd_lat_kernel, MODE 0, beside the tiles it stages)
//   dz_m    = sum_n Bt[n,m] dy_n                   (bwd_lat_kernel, MODE 0; split over N + merge)
//   Delta_m = <dz_m, z_m>                          (merge)
//   dS[m,n] = A (<dz_m,v_n> - Delta_m) + Bt (<dy_n,z_m> - delta_n)
//   dv_n    = sum_m A[m,n] dz_m ;  dk_n = s sum_m dS[m,n] q_m      (bwd_tok_kernel, token parallel)
//   dq_m    = s sum_n dS[m,n] k_n                  (bwd_lat_kernel, MODE 1; split over N + merge)
// The additive terms (-L_m, -rho_n, -Delta_m, -delta_n) enter as the initial accumulator of the
// matrix product they belong to wherever the tile layout gives them for free (a row vector of the
// tile), instead of one subtraction per element.
// Both exponentials are bounded by 1, so no running maximum is needed anywhere.  The two kernel
// shapes are those of the forward: "latent side" = the gather's (K/V/dY tiles of 64 tokens in LDS,
// lane = latent, contraction over tokens), "token side" = the scatter's (latent operands in LDS,
// lane = token, contraction over latents).  Score-like products <.,.> run on v_mfma_f32_16x16x32
// exactly like the scores; their fp32 tiles line up element by element with the score tile, so dS
// is assembled in registers and, packed to bf16, is the B operand of the last product.
// q and k meet in the element type; every other product runs in bf16 (f16 tiles are converted while
// they are staged), because dz, Delta and dS have no useful bound in f16.
//
// One exponential per score instead of two.  Both weights come from the same score, so
//   Bt[n,m] = A[m,n] * eL[m] * eR[n],   eL[m] = exp2(L2_m - Lmax2) <= 1,   eR[n] = exp2(Lmax2 - rho2_n)
// (log2 units, Lmax2 = the largest L2_m of the (b,h)).  The kernels that need both weights fold eR into the rows of
// dy and into delta_n when they load a token tile, and eL into a per-latent factor, and evaluate
//   dS = A * (<dz_m,v_n> - Delta_m + eL[m] * (<z_m, eR dy_n> - eR delta_n)).
// That is exact unless A underflows where Bt still matters or eR overflows, which needs log-sum-exps more than
// kFactorSpan apart: the dz pass records the smallest rho2_n of every split, and a (b,h) whose Lmax2 exceeds the
// smallest rho2_n by more than kFactorSpan takes the two-exponential form for all its tiles.
// (Padded tokens and empty batch elements carry log-sum-exps of 1e30: the former are ignored by the minimum and
// get eR = 0, the latter send their (b,h) to the two-exponential form.)
//
// Attention dropout of the forward (MixerBwdArgs::drop_thr != 0): the keep masks are regenerated from the same hash.  With
// K1, K2 the keep factors (0 or 1 / (1 - p)) of the two phases the forward used K1 A and K2 Bt, so
//   dz_m = sum_n K2 Bt dy_n,  dv_n = sum_m K1 A dz_m,  dS = A (K1 <dz_m,v_n> - Delta_m) + Bt (K2 <dy_n,z_m> - delta_n)
// with the same Delta_m = <dz_m, z_m> and delta_n = <dy_n, y_n> (sums over the kept weights already).  These problems
// take the two-exponential form with every additive term applied element by element.
#include <algorithm>
#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mb;
template <> struct Mb<bf16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float unpack(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
};
template <> struct Mb<f16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float unpack(uint16_t b) { return float(__builtin_bit_cast(_Float16, b)); }
};
using Pb = Mb<bf16_t>;

__device__ __forceinline__ u32x4 zero4() { return u32x4{0u, 0u, 0u, 0u}; }
__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }

// 8 packed elements of type T scaled by f, repacked in T
template <typename T> __device__ __forceinline__ u32x4 scale8(u32x4 v, float f)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = Mb<T>::pack2(Mb<T>::unpack(uint16_t(v[i] & 0xffffu)) * f, Mb<T>::unpack(uint16_t(v[i] >> 16)) * f);
    return o;
}
// 8 packed elements of type T scaled by f, as packed bf16
template <typename T> __device__ __forceinline__ u32x4 to_bf16x8(u32x4 v, float f = 1.f)
{
    if (std::is_same<T, bf16_t>::value && f == 1.f) return v;
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = Pb::pack2(Mb<T>::unpack(uint16_t(v[i] & 0xffffu)) * f, Mb<T>::unpack(uint16_t(v[i] >> 16)) * f);
    return o;
}
// 8 consecutive fp32 values as packed bf16
__device__ __forceinline__ u32x4 pack8(const float* p)
{
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
    return u32x4{Pb::pack2(a[0], a[1]), Pb::pack2(a[2], a[3]), Pb::pack2(b[0], b[1]), Pb::pack2(b[2], b[3])};
}
__device__ __forceinline__ u32x4 pack8(const float (&v)[8])
{
    return u32x4{Pb::pack2(v[0], v[1]), Pb::pack2(v[2], v[3]), Pb::pack2(v[4], v[5]), Pb::pack2(v[6], v[7])};
}
// 8 consecutive fp32 values times f as packed bf16
__device__ __forceinline__ u32x4 pack8(const float* p, float f)
{
    const f32x4 a = *reinterpret_cast<const f32x4*>(p) * f, b = *reinterpret_cast<const f32x4*>(p + 4) * f;
    return u32x4{Pb::pack2(a[0], a[1]), Pb::pack2(a[2], a[3]), Pb::pack2(b[0], b[1]), Pb::pack2(b[2], b[3])};
}

// Largest distance (log2 units) between the latents' largest log-sum-exp and a token's for which the token
// scatter's weights are formed from the gather's (see the head of this file): exp2(64) and the 2^-62 that is
// left of a weight whose partner underflowed are both far inside what fp32 and bf16 hold.
constexpr float kFactorSpan = 64.f;

__device__ __forceinline__ float wave_max(float x)
{
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
    return x;
}

// Whether the (b,h) may use the one-exponential form, and its Lmax2.  Every wave computes the same answer.
__device__ __forceinline__ bool factor_plan(const MixerBwdArgs& a, int64_t bh, int lane, float& lmax2)
{
    float lm = -3.0e38f, rm = -3.0e38f;
    for (int m = lane; m < a.M; m += 64) lm = fmaxf(lm, a.lse_lat[bh * a.M + m]);
    for (int p = lane; p < a.n_splits0; p += 64) rm = fmaxf(rm, -a.rho_min[bh * a.n_splits0 + p]);
    lmax2 = wave_max(lm) * kLog2e;
    // An empty batch element (its latents carry 1e30) takes the other form: differences of such magnitudes are
    // rounding noise far above the range of exp2.
    return lmax2 <= 1.0e6f && lmax2 + wave_max(rm) <= kFactorSpan;
}

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

// <u, w> of eight 16-bit elements
template <typename T>
__device__ __forceinline__ float dot8(u32x4 u, u32x4 w)
{
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        s = fmaf(Mb<T>::unpack(uint16_t(u[i] & 0xffffu)), Mb<T>::unpack(uint16_t(w[i] & 0xffffu)), s);
        s = fmaf(Mb<T>::unpack(uint16_t(u[i] >> 16)), Mb<T>::unpack(uint16_t(w[i] >> 16)), s);
    }
    return s;
}

// ---- latent side ---------------------------------------------------------------------------
constexpr int kBTile = 64;   // tokens per LDS tile

// One workgroup = 4 waves x (16 CT latents) x one token range.  MODE 0: dz partial; MODE 1: dq partial.
template <typename T, int D, int CT, int MODE, bool DROPK>
__global__ __launch_bounds__(256, MODE == 1 ? bwd_dq_wgs_per_cu(D, CT) : 2) void bwd_lat_kernel(MixerBwdArgs a)
{
    constexpr int KD = (D + 31) / 32, RT = D / 16, CH = D / 8, MB = 64 * CT, ROWB = D * 2, TILEB = kBTile * ROWB;
    constexpr int NT = MODE == 0 ? 2 : 4;          // staged tiles: K rows, dY^T | K rows, K^T, V rows, dY rows
    using M_ = Mb<T>;
    __shared__ __attribute__((aligned(16))) uint8_t tl[2][NT][TILEB];
    __shared__ __attribute__((aligned(16))) float tsc[2][2][kBTile];   // per-token scalars of a tile: -rho * log2(e), -delta

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int mblocks = (a.M + MB - 1) / MB;     // M % 64 == 32: waves 2, 3 of the last block own no latent, they only help stage
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;
    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint16_t* dy = (const uint16_t*)a.dy + b * a.dys[0] + h * a.dys[1];
    const uint16_t* yv = (const uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    const float* rho = a.lse_tok + bh * a.N;
    float* dlt = a.delta_tok + bh * a.N;
    const int m_base = mb * MB + w * 16 * CT;
    // The dz pass also produces delta_n = <dy_n, y_n> for the later passes: its first latent block
    // reads the rows of y next to those of dy, which it stages anyway.
    const bool make_delta = MODE == 0 && mb == 0;

    // the dq pass forms the token scatter's weights from the gather's where the (b,h) allows it
    // (a forward with attention dropout: the two weights meet different keep masks, which the one-exponential form,
    // one accumulator for both inner products, cannot apply)
    float lmax2 = 0.f;
    const bool fast = MODE == 1 && !DROPK && factor_plan(a, bh, lane, lmax2);

    // latent operands (B of the score-like products) and per-latent scalars
    u32x4 qb[CT][KD], dzb[CT][KD], zb[CT][KD];
    float nel[CT];                                  // -eL[m] of the lane's latent (one-exponential form)
    // The additive terms of the score-like products (-L_m, -rho_n, -Delta_m, -delta_n) are not
    // subtracted element by element: they are the initial accumulator of the matrix product.  A
    // per-token term is a row vector of the tile (free); a per-latent term needs four registers
    // holding the same value, which the register budget allows up to D = 32.
    constexpr bool kFoldLat = MODE == 1 && D <= 32;
    float l2m[CT], dm[CT];
    f32x4 nl4[kFoldLat ? CT : 1], nd4[kFoldLat ? CT : 1];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = m_base + ct * 16 + c16;
        const bool own = m_base + ct * 16 < a.M;       // uniform over the wave
        // eL[m]: the rows of z carry it in the one-exponential form (1 otherwise)
        const float el = (MODE == 1 && fast && own) ? fast_exp2(a.lse_lat[bh * a.M + m] * kLog2e - lmax2) : 1.f;
        nel[ct] = -el;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const int ch = kd * 4 + g;
            const bool in = own && ch < CH;
            qb[ct][kd] = in ? scale8<T>(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2) : zero4();
            if (MODE == 1) {
                dzb[ct][kd] = in ? pack8(a.dz + (bh * a.M + m) * D + ch * 8) : zero4();
                zb[ct][kd] = in ? pack8(a.z + (bh * a.M + m) * D + ch * 8, el) : zero4();
            }
        }
        if (MODE == 1) {
            l2m[ct] = own ? a.lse_lat[bh * a.M + m] * kLog2e : 0.f;
            dm[ct] = own ? a.delta_lat[bh * a.M + m] : 0.f;
            if constexpr (kFoldLat) {
                nl4[ct] = f32x4{-l2m[ct], -l2m[ct], -l2m[ct], -l2m[ct]};
                nd4[ct] = f32x4{-dm[ct], -dm[ct], -dm[ct], -dm[ct]};
            }
        }
    }

    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);

    constexpr int TCH = kBTile * CH;
    constexpr int CPT = (TCH + 255) / 256;
    auto k_slot = [](int tok, int ch) { return tok * ROWB + ((ch ^ ((tok >> 2) & (CH - 1))) << 4); };
    auto v_slot = [](int tok, int ch) { return tok * ROWB + ((CH >= 4 ? (ch ^ (((tok >> 2) & 1) << 1)) : ch) << 4); };

    u32x4 kr[CPT], vr[CPT], yr[CPT];
    float ysc[CPT];    // eR of the token a staged dy chunk belongs to (one-exponential form)
    float rr = 0.f, dd = 0.f;
    float rr_max = -3.0e38f;   // MODE 0: -(smallest rho2_n) over the tokens this thread has loaded
    int ln0 = 0;       // first token of the tile held in kr/vr/yr
    auto load_tile = [&](int n0) {
        ln0 = n0;
        if (tid < kBTile) {
            const int n = min(n0 + tid, n_end - 1);
            rr = -rho[n] * kLog2e;          // negated: they start the accumulators of the products below
            if (MODE == 0) rr_max = fmaxf(rr_max, rr);
            if (MODE == 1) dd = fast ? dlt[n] * fast_exp2(lmax2 + rr) : -dlt[n];     // eR delta_n | -delta_n
        }
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * 256;
            ysc[i] = 1.f;
            if (c < TCH) {
                const int n = min(n0 + c / CH, n_end - 1), ch = c % CH;
                if (MODE == 1 && fast) ysc[i] = fast_exp2(lmax2 - rho[n] * kLog2e);
                kr[i] = load16(k + (int64_t)n * a.ks[2] + ch * 8);
                yr[i] = load16(dy + (int64_t)n * a.dys[2] + ch * 8);
                if (MODE == 1) vr[i] = load16(v + (int64_t)n * a.vs[2] + ch * 8);
                if (MODE == 0 && make_delta) vr[i] = load16(yv + (int64_t)n * a.ys[2] + ch * 8);
            }
        }
    };
    auto store_tile = [&](int buf) {
        if (tid < kBTile) {
            tsc[buf][0][tid] = rr;
            tsc[buf][1][tid] = dd;
        }
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * 256;
            if (c < TCH) {
                const int tok = c / CH, ch = c % CH;
                *reinterpret_cast<u32x4*>(&tl[buf][0][k_slot(tok, ch)]) = kr[i];
                if (MODE == 0) {
                    *reinterpret_cast<u32x4*>(&tl[buf][1][v_slot(tok, ch)]) = to_bf16x8<T>(yr[i]);
                    if (make_delta) {      // uniform over the workgroup; the CH lanes of a token are neighbours
                        float pd = dot8<T>(yr[i], vr[i]);
#pragma unroll
                        for (int o = 1; o < CH; o <<= 1) pd += __shfl_xor(pd, o);
                        if (ch == 0 && ln0 + tok < n_end) dlt[ln0 + tok] = pd;
                    }
                } else {
                    *reinterpret_cast<u32x4*>(&tl[buf][1][v_slot(tok, ch)]) = to_bf16x8<T>(kr[i]);
                    *reinterpret_cast<u32x4*>(&tl[buf][2][k_slot(tok, ch)]) = to_bf16x8<T>(vr[i]);
                    *reinterpret_cast<u32x4*>(&tl[buf][3][k_slot(tok, ch)]) = to_bf16x8<T>(yr[i], ysc[i]);
                }
            }
        }
    };

    f32x4 acc[RT][CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 zf = {0.f, 0.f, 0.f, 0.f};

    auto process = [&](auto fast_c, auto drop_c, int n0, int buf) {
        constexpr bool FAST = decltype(fast_c)::value;      // one-exponential form (dq pass only)
        // DROP: the forward dropped weights.  Every additive term is then applied element by element (accumulators start
        // at zero), because the inner products meet their keep factors before the row sums are subtracted:
        // dS = A (K1 <dz,v> - Delta) + B (K2 <dy,z> - delta), and dz = sum_n K2 B dy.
        constexpr bool DROP = decltype(drop_c)::value;
        constexpr bool FoldLat = kFoldLat && !DROP;
        const bool full = n0 + kBTile <= n_end;
#pragma unroll
        for (int ks = 0; ks < kBTile / 32; ++ks) {
            u32x4 ka0[KD], ka1[KD], va0[KD], va1[KD], ya0[KD], ya1[KD], tr[RT];
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                const int ch = kd * 4 + g, t0 = ks * 32 + c16, t1 = t0 + 16;
                ka0[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&tl[buf][0][k_slot(t0, ch)]) : zero4();
                ka1[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&tl[buf][0][k_slot(t1, ch)]) : zero4();
                if (MODE == 1) {
                    va0[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&tl[buf][2][k_slot(t0, ch)]) : zero4();
                    va1[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&tl[buf][2][k_slot(t1, ch)]) : zero4();
                    ya0[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&tl[buf][3][k_slot(t0, ch)]) : zero4();
                    ya1[kd] = ch < CH ? *reinterpret_cast<const u32x4*>(&tl[buf][3][k_slot(t1, ch)]) : zero4();
                }
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                // transposed tile (dY^T or K^T): rows d, k-slots = the 8 tokens of this lane group
                const int r0 = ks * 32 + 4 * g + (c16 >> 2), r1 = r0 + 16;
                const int ch = 2 * rt + ((c16 & 3) >> 1), sub = (c16 & 1) << 3;
                const uint2 lo = lds_read_tr16(&tl[buf][1][v_slot(r0, ch) + sub]);
                const uint2 hi = lds_read_tr16(&tl[buf][1][v_slot(r1, ch) + sub]);
                tr[rt] = u32x4{lo.x, lo.y, hi.x, hi.y};
            }
            // negated per-token scalars of the 8 tokens (rows) this lane holds: 4g .. 4g+3 and 16+4g .. 16+4g+3
            const int tb = ks * 32 + 4 * g;
            const f32x4 ra = *reinterpret_cast<const f32x4*>(&tsc[buf][0][tb]), rb = *reinterpret_cast<const f32x4*>(&tsc[buf][0][tb + 16]);
            f32x4 da = zf, db = zf;
            if (MODE == 1) {
                da = *reinterpret_cast<const f32x4*>(&tsc[buf][1][tb]);
                db = *reinterpret_cast<const f32x4*>(&tsc[buf][1][tb + 16]);
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                float o[8];
                if constexpr (FAST) {
                    // A = exp2(S - L_m);  g = <dz_m,v_n> - Delta_m + <eL z_m, eR dy_n>;  dS = A (g - eL[m] eR delta_n)
                    f32x4 a0 = kFoldLat ? nl4[kFoldLat ? ct : 0] : zf, a1 = a0;
                    f32x4 g0 = kFoldLat ? nd4[kFoldLat ? ct : 0] : zf, g1 = g0;
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        a0 = M_::mma(ka0[kd], qb[ct][kd], a0);
                        a1 = M_::mma(ka1[kd], qb[ct][kd], a1);
                        g0 = Pb::mma(va0[kd], dzb[ct][kd], g0);
                        g1 = Pb::mma(va1[kd], dzb[ct][kd], g1);
                    }
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        g0 = Pb::mma(ya0[kd], zb[ct][kd], g0);
                        g1 = Pb::mma(ya1[kd], zb[ct][kd], g1);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if constexpr (kFoldLat) {
                            o[e] = fast_exp2(a0[e]) * fmaf(nel[ct], da[e], g0[e]);
                            o[e + 4] = fast_exp2(a1[e]) * fmaf(nel[ct], db[e], g1[e]);
                        } else {
                            o[e] = fast_exp2(a0[e] - l2m[ct]) * (fmaf(nel[ct], da[e], g0[e]) - dm[ct]);
                            o[e + 4] = fast_exp2(a1[e] - l2m[ct]) * (fmaf(nel[ct], db[e], g1[e]) - dm[ct]);
                        }
                    }
                    if (!full) {       // rows past the end of the token range (clamped copies of the last token)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (n0 + tb + e >= n_end) o[e] = 0.f;
                            if (n0 + tb + 16 + e >= n_end) o[e + 4] = 0.f;
                        }
                    }
                    const u32x4 obf = pack8(o);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[rt][ct] = Pb::mma(tr[rt], obf, acc[rt][ct]);
                    continue;
                }
                // S - rho_n: the token scatter's exponent
                constexpr bool kFoldTok = (MODE == 0 || kFoldLat) && !DROP;
                f32x4 b0 = kFoldTok ? ra : zf, b1 = kFoldTok ? rb : zf;
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) {
                    b0 = M_::mma(ka0[kd], qb[ct][kd], b0);
                    b1 = M_::mma(ka1[kd], qb[ct][kd], b1);
                }
                // keep factors (0 or 1 / (1 - p)) of the lane's eight entries: gather's weights, scatter's weights
                float k1[DROP ? 8 : 1], k2[DROP ? 8 : 1];
                if constexpr (DROP) {
                    const uint32_t m = (uint32_t)(m_base + ct * 16 + c16);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const uint32_t n = (uint32_t)(n0 + tb + (e >> 2) * 16 + (e & 3));
                        if (MODE == 1) k1[e] = dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 0u, (uint32_t)bh, m, n);
                        k2[e] = dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 1u, (uint32_t)bh, m, n);
                    }
                }
                if (MODE == 0) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if constexpr (DROP) {
                            o[e] = fast_exp2(b0[e] + ra[e]) * k2[e];
                            o[e + 4] = fast_exp2(b1[e] + rb[e]) * k2[e + 4];
                        } else {
                            o[e] = fast_exp2(b0[e]);
                            o[e + 4] = fast_exp2(b1[e]);
                        }
                    }
                } else {
                    // S - L_m (the latent gather's exponent), <dz_m, v_n> - Delta_m and <dy_n, z_m> - delta_n
                    f32x4 a0 = FoldLat ? nl4[kFoldLat ? ct : 0] : zf, a1 = a0;
                    f32x4 g10 = FoldLat ? nd4[kFoldLat ? ct : 0] : zf, g11 = g10, g20 = FoldLat ? da : zf, g21 = FoldLat ? db : zf;
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        if constexpr (FoldLat) {
                            a0 = M_::mma(ka0[kd], qb[ct][kd], a0);
                            a1 = M_::mma(ka1[kd], qb[ct][kd], a1);
                        }
                        g10 = Pb::mma(va0[kd], dzb[ct][kd], g10);
                        g11 = Pb::mma(va1[kd], dzb[ct][kd], g11);
                        g20 = Pb::mma(ya0[kd], zb[ct][kd], g20);
                        g21 = Pb::mma(ya1[kd], zb[ct][kd], g21);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if constexpr (DROP) {
                            o[e] = fast_exp2(b0[e] - l2m[ct]) * (k1[e] * g10[e] - dm[ct]) + fast_exp2(b0[e] + ra[e]) * (k2[e] * g20[e] + da[e]);
                            o[e + 4] = fast_exp2(b1[e] - l2m[ct]) * (k1[e + 4] * g11[e] - dm[ct]) +
                                       fast_exp2(b1[e] + rb[e]) * (k2[e + 4] * g21[e] + db[e]);
                        } else if constexpr (kFoldLat) {
                            o[e] = fast_exp2(a0[e]) * g10[e] + fast_exp2(b0[e]) * g20[e];
                            o[e + 4] = fast_exp2(a1[e]) * g11[e] + fast_exp2(b1[e]) * g21[e];
                        } else {    // plain products; every term is applied element by element
                            o[e] = fast_exp2(b0[e] - l2m[ct]) * (g10[e] - dm[ct]) + fast_exp2(b0[e] + ra[e]) * (g20[e] + da[e]);
                            o[e + 4] = fast_exp2(b1[e] - l2m[ct]) * (g11[e] - dm[ct]) + fast_exp2(b1[e] + rb[e]) * (g21[e] + db[e]);
                        }
                    }
                }
                if (!full) {       // rows past the end of the token range (clamped copies of the last token)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n0 + tb + e >= n_end) o[e] = 0.f;
                        if (n0 + tb + 16 + e >= n_end) o[e + 4] = 0.f;
                    }
                }
                const u32x4 ob = pack8(o);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) acc[rt][ct] = Pb::mma(tr[rt], ob, acc[rt][ct]);
            }
        }
    };

    if (n_begin < n_end) {
        load_tile(n_begin);
        store_tile(0);
    }
    __syncthreads();
    auto walk = [&](auto fast_c, auto drop_c) {
        int buf = 0;
        for (int n0 = n_begin; n0 < n_end; n0 += kBTile, buf ^= 1) {
            const bool more = n0 + kBTile < n_end;
            if (more) load_tile(n0 + kBTile);
            process(fast_c, drop_c, n0, buf);
            if (more) store_tile(buf ^ 1);
            __syncthreads();
        }
    };
    if constexpr (DROPK) {
        walk(std::false_type{}, std::true_type{});
    } else if constexpr (MODE == 1) {
        if (fast) walk(std::true_type{}, std::false_type{});
        else walk(std::false_type{}, std::false_type{});
    } else {
        walk(std::false_type{}, std::false_type{});
    }

    if (make_delta) {
        // the smallest token log-sum-exp of this split (log2 units), for the passes that follow
        const float rm = wave_max(rr_max);      // wave 0 = the threads that read the tokens' scalars
        if (tid == 0) a.rho_min[bh * a.n_splits + split] = -rm;
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = m_base + ct * 16 + c16;
        if (m >= a.M) continue;
        const int64_t row = ((int64_t)bh * a.n_splits + split) * a.M + m;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) *reinterpret_cast<f32x4*>(a.part + row * D + rt * 16 + 4 * g) = acc[rt][ct];
    }
}

// MODE 0: dz = sum of partials, Delta_m = <dz_m, z_m>;  MODE 1: dq = scale * sum of partials.
// One thread per (b,h,m) and four channels; the partials are summed in split order (bit-stable).
template <int MODE>
__global__ __launch_bounds__(256) void bwd_merge_kernel(MixerBwdArgs a)
{
    const int dq4 = a.D / 4;                                       // threads per row: 4, 8 or 16
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t rows = (int64_t)a.B * a.H * a.M;
    const bool live = t < rows * dq4;
    const int64_t r = live ? t / dq4 : rows - 1;                   // (b*H + h)*M + m
    const int d = (int)(t % dq4) * 4;
    const int m = r % a.M;
    const int64_t bh = r / a.M;
    const float* p0 = a.part + (bh * a.n_splits * a.M + m) * a.D + d;
    const int64_t sp = (int64_t)a.M * a.D;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8      // eight loads in flight; the additions keep the split order
    for (int p = 0; p < a.n_splits; ++p) s += *reinterpret_cast<const f32x4*>(p0 + p * sp);
    if (MODE == 0) {
        const f32x4 zz = *reinterpret_cast<const f32x4*>(a.z + r * a.D + d);
        float delta = s[0] * zz[0] + s[1] * zz[1] + s[2] * zz[2] + s[3] * zz[3];
        for (int o = 1; o < dq4; o <<= 1) delta += __shfl_xor(delta, o);   // the threads of a row are neighbours
        if (live) {
            *reinterpret_cast<f32x4*>(a.dz + r * a.D + d) = s;
            // scatter half alone: the array stands in for lse_lat there and keeps the value that switches the gather term off
            if (d == 0 && a.half != 2) a.delta_lat[r] = delta;
        }
    } else if (live) {
        *reinterpret_cast<f32x4*>(a.dq + r * a.D + d) = s * a.scale;
    }
}

// The halves of the mixer differentiated alone run the whole mixer's kernels with the other half's softmax weights
// forced to zero: a log-sum-exp of 1e30 makes exp2(S - 1.44e30) vanish, and every term that multiplies it stays
// finite.  Gather half (a.half == 1, dz given): lse_tok, delta_tok (one array) and rho_min are filled with 1e30 and
// Delta_m = <dz_m, z_m> is formed here instead of in the dz pass's merge.  Scatter half (a.half == 2): delta_lat, which
// stands in for lse_lat, is filled with 1e30 (that batch element then takes the two-exponential form).
__global__ __launch_bounds__(256) void bwd_half_prep_kernel(MixerBwdArgs a)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x, step = (int64_t)gridDim.x * 256;
    const int64_t lat = (int64_t)a.B * a.H * a.M;
    if (a.half == 2) {
        for (int64_t i = t; i < lat; i += step) a.delta_lat[i] = 1.0e30f;
        return;
    }
    for (int64_t i = t; i < (int64_t)a.B * a.H * a.N; i += step) a.delta_tok[i] = 1.0e30f;
    for (int64_t i = t; i < (int64_t)a.B * a.H * a.n_splits0; i += step) a.rho_min[i] = 1.0e30f;
    for (int64_t r = t; r < lat; r += step) {
        float s = 0.f;
        for (int d = 0; d < a.D; d += 4) {
            const f32x4 x = *reinterpret_cast<const f32x4*>(a.dz + r * a.D + d), y = *reinterpret_cast<const f32x4*>(a.z + r * a.D + d);
            s += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
        }
        a.delta_lat[r] = s;
    }
}

// ---- token side ----------------------------------------------------------------------------

// The five latent-side operand sets fill most of a CU's LDS at the usual sizes (82 KB at M = 256,
// D = 32), so only one workgroup fits: it has 8 waves, two per SIMD, all reading the same operands.
template <int D> constexpr int kTokWaves = D <= 32 ? 12 : 8;
template <int D> constexpr int kTokTiles = 2;      // 16-token column tiles per wave iteration

template <typename T, int D, bool DROPK>
__global__ __launch_bounds__(64 * kTokWaves<D>, 1) void bwd_tok_kernel(MixerBwdArgs a, int tokens_per_wg)
{
    constexpr int NTH = 64 * kTokWaves<D>;
    constexpr int KD = (D + 31) / 32, RT = D / 16, CH = D / 8;
    constexpr int kBTW = kTokTiles<D>;
    using M_ = Mb<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // M here is the chunk of latents this launch covers: when the five operand sets of all latents exceed the LDS,
    // the launch is repeated over chunks and every launch after the first adds to dk, dv
    const int M = a.mc > 0 ? a.mc : a.M, KS = M / 32;
    // A-operand layout [mt][ch][c16] for q (scaled, log2 units), dz, z;  PV-operand layout
    // [ks][rt][lane] for dz^T and (scale q)^T;  per-latent scalars
    u32x4* qa = reinterpret_cast<u32x4*>(smem);
    u32x4* dza = qa + (size_t)M * CH;
    u32x4* zza = dza + (size_t)M * CH;
    u32x4* dzt = zza + (size_t)M * CH;
    u32x4* qt = dzt + (size_t)M * CH;
    // The per-latent scalars (-L2_m, -Delta_m, -eL[m]) sit behind the operand sets when the LDS has room for them
    // (a.scal_lds); when the five operand sets take all 160 KB (M = 256 at D = 64, M = 512 at D = 32) they are read
    // from global memory at every latent step.
    float* sc_l = reinterpret_cast<float*>(qt + (size_t)M * CH);     // [3][M] when a.scal_lds
    const float* lse_lat = a.lse_lat + ((int64_t)blockIdx.z * a.H + blockIdx.y) * a.M + a.m0;
    const float* delta_lat = a.delta_lat + ((int64_t)blockIdx.z * a.H + blockIdx.y) * a.M + a.m0;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;
    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1] + (int64_t)a.m0 * a.qs[2];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const uint16_t* dy = (const uint16_t*)a.dy + b * a.dys[0] + h * a.dys[1];
    uint16_t* dk = (uint16_t*)a.dk + b * a.dks[0] + h * a.dks[1];
    uint16_t* dv = (uint16_t*)a.dv + b * a.dvs[0] + h * a.dvs[1];
    const float* z = a.z + (bh * a.M + a.m0) * D;
    const float* dz = a.dz + (bh * a.M + a.m0) * D;
    const float* rho = a.lse_tok + bh * a.N;
    const float* dlt = a.delta_tok + bh * a.N;

    float lmax2 = 0.f;
    const bool fast = !DROPK && factor_plan(a, (int64_t)blockIdx.z * a.H + blockIdx.y, threadIdx.x & 63, lmax2);
    if (a.only_form == 2) {     // the 32x32x16 token pass has taken the (b,h) of the unshifted form
        float unused;
        if (bwd_unshifted_form(a, (int64_t)blockIdx.z * a.H + blockIdx.y, threadIdx.x & 63, unused)) return;
    }
    if (a.scal_lds) {
        for (int m = threadIdx.x; m < M; m += NTH) {
            const float l2 = lse_lat[m] * kLog2e;
            sc_l[m] = -l2;
            sc_l[M + m] = -delta_lat[m];
            sc_l[2 * M + m] = -fast_exp2(l2 - lmax2);
        }
    }
    for (int idx = tid; idx < M * CH; idx += NTH) {
        const int m = idx / CH, ch = idx % CH;
        const int slot = ((m >> 4) * CH + ch) * 16 + (m & 15);
        qa[slot] = scale8<T>(load16(q + (int64_t)m * a.qs[2] + ch * 8), a.scale_log2);
        dza[slot] = pack8(dz + (int64_t)m * D + ch * 8);
        // the rows of z carry eL[m] in the one-exponential form
        zza[slot] = pack8(z + (int64_t)m * D + ch * 8, fast ? fast_exp2(lse_lat[m] * kLog2e - lmax2) : 1.f);
    }
    for (int idx = tid; idx < KS * RT * 64; idx += NTH) {
        const int ln = idx & 63, rt = (idx >> 6) % RT, ks = idx / (64 * RT);
        const int cc = ln & 15, gg = ln >> 4;
        const int d = (D / 4) * (cc >> 2) + 4 * rt + (cc & 3);
        u32x4 o1, o2;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            const int e = 2 * e2;
            const int m0 = 32 * ks + (e >> 2) * 16 + 4 * gg + (e & 3);
            o1[e2] = Pb::pack2(dz[(int64_t)m0 * D + d], dz[(int64_t)(m0 + 1) * D + d]);
            o2[e2] = Pb::pack2(M_::unpack(q[(int64_t)m0 * a.qs[2] + d]) * a.scale, M_::unpack(q[(int64_t)(m0 + 1) * a.qs[2] + d]) * a.scale);
        }
        dzt[idx] = o1;
        qt[idx] = o2;
    }
    __syncthreads();

    const int wg_n0 = blockIdx.x * tokens_per_wg;
    const int wg_n1 = min(a.N, wg_n0 + tokens_per_wg);
    const f32x4 zf = {0.f, 0.f, 0.f, 0.f};

    // FAST = the one-exponential form (head of this file): the rows of dy and delta_n carry eR[n], the element-wise
    // part applies eL[m]; otherwise both exponentials are taken.
    // DROP = the forward dropped weights: -Delta_m leaves the accumulator of <dz, v> and is applied after the keep factor,
    // dS = A (K1 <dz,v> - Delta) + B (K2 <dy,z> - delta), and dv meets K1 A.
    auto walk = [&](auto fast_c, auto drop_c, const float lmax2) {
    constexpr bool FAST = decltype(fast_c)::value;
    constexpr bool DROP = decltype(drop_c)::value;
    for (int t0 = wg_n0 + w * 16 * kBTW; t0 < wg_n1; t0 += kTokWaves<D> * 16 * kBTW) {
        u32x4 kb[kBTW][KD], vb[kBTW][KD], yb[kBTW][KD];
        float r2[kBTW], de[kBTW];      // FAST: r2 is unused, de = eR delta_n
#pragma unroll
        for (int tw = 0; tw < kBTW; ++tw) {
            const int n = t0 + tw * 16 + c16;
            const bool live = n < wg_n1;
            const int nc = live ? n : wg_n1 - 1;
            r2[tw] = rho[nc] * kLog2e;
            const float er = FAST ? fast_exp2(lmax2 - r2[tw]) : 1.f;
            de[tw] = dlt[nc] * er;
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                const int ch = kd * 4 + g;
                const bool in = live && ch < CH;
                kb[tw][kd] = in ? load16(k + (int64_t)n * a.ks[2] + ch * 8) : zero4();
                vb[tw][kd] = in ? to_bf16x8<T>(load16(v + (int64_t)n * a.vs[2] + ch * 8)) : zero4();
                yb[tw][kd] = in ? to_bf16x8<T>(load16(dy + (int64_t)n * a.dys[2] + ch * 8), er) : zero4();
            }
        }
        f32x4 adk[kBTW][RT], adv[kBTW][RT];
#pragma unroll
        for (int tw = 0; tw < kBTW; ++tw)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) adk[tw][rt] = adv[tw][rt] = zf;

        for (int ks = 0; ks < KS; ++ks) {
            u32x4 q0[KD], q1[KD], d0[KD], d1[KD], z0[KD], z1[KD], odz[RT], oq[RT];
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                const int ch = kd * 4 + g;
                const int s0 = ((2 * ks) * CH + ch) * 16 + c16, s1 = ((2 * ks + 1) * CH + ch) * 16 + c16;
                q0[kd] = ch < CH ? qa[s0] : zero4();
                q1[kd] = ch < CH ? qa[s1] : zero4();
                d0[kd] = ch < CH ? dza[s0] : zero4();
                d1[kd] = ch < CH ? dza[s1] : zero4();
                z0[kd] = ch < CH ? zza[s0] : zero4();
                z1[kd] = ch < CH ? zza[s1] : zero4();
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                odz[rt] = dzt[(ks * RT + rt) * 64 + lane];
                oq[rt] = qt[(ks * RT + rt) * 64 + lane];
            }
            // negated per-latent scalars of the 8 latents (rows) this lane holds: -L_m log2(e) and -Delta_m
            // start the accumulators of S and <dz, v>, so neither is subtracted element by element
            f32x4 la, lb, da, db, nea = zf, neb = zf;      // -L2_m, -Delta_m, -eL[m] of the 8 latents (rows) this lane holds
            if (a.scal_lds) {
                const float* t = sc_l + 32 * ks + 4 * g;
                la = *reinterpret_cast<const f32x4*>(t);            lb = *reinterpret_cast<const f32x4*>(t + 16);
                da = *reinterpret_cast<const f32x4*>(t + M);        db = *reinterpret_cast<const f32x4*>(t + M + 16);
                if (FAST) {
                    nea = *reinterpret_cast<const f32x4*>(t + 2 * M);
                    neb = *reinterpret_cast<const f32x4*>(t + 2 * M + 16);
                }
            } else {
                la = *reinterpret_cast<const f32x4*>(lse_lat + 32 * ks + 4 * g) * -kLog2e;
                lb = *reinterpret_cast<const f32x4*>(lse_lat + 32 * ks + 16 + 4 * g) * -kLog2e;
                da = -*reinterpret_cast<const f32x4*>(delta_lat + 32 * ks + 4 * g);
                db = -*reinterpret_cast<const f32x4*>(delta_lat + 32 * ks + 16 + 4 * g);
                if (FAST) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        nea[e] = -fast_exp2(-la[e] - lmax2);
                        neb[e] = -fast_exp2(-lb[e] - lmax2);
                    }
                }
            }
            if constexpr (FAST) {
                // The rows of z carry eL[m] (staged that way when the (b,h) takes this form), so
                //   g = <dz_m,v_n> - Delta_m + <eL z_m, eR dy_n>   is one accumulator chain,   dS = A (g - eL[m] eR delta_n).
                // Software pipeline over the wave's tiles: the score-like products of tile tw + 1 and the gradient
                // products of tile tw - 1 are issued ahead of the exponentials of tile tw, which run under them.
                auto front = [&](int tw, f32x4& a0, f32x4& a1, f32x4& g0, f32x4& g1) {
                    a0 = la; a1 = lb; g0 = da; g1 = db;
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        a0 = M_::mma(q0[kd], kb[tw][kd], a0);
                        a1 = M_::mma(q1[kd], kb[tw][kd], a1);
                        g0 = Pb::mma(d0[kd], vb[tw][kd], g0);
                        g1 = Pb::mma(d1[kd], vb[tw][kd], g1);
                    }
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        g0 = Pb::mma(z0[kd], yb[tw][kd], g0);
                        g1 = Pb::mma(z1[kd], yb[tw][kd], g1);
                    }
                };
                auto back = [&](int tw, u32x4 pa, u32x4 pd) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        adv[tw][rt] = Pb::mma(odz[rt], pa, adv[tw][rt]);
                        adk[tw][rt] = Pb::mma(oq[rt], pd, adk[tw][rt]);
                    }
                };
                f32x4 a0, a1, g0, g1;
                front(0, a0, a1, g0, g1);
                u32x4 pap = zero4(), pdp = zero4();
#pragma unroll
                for (int tw = 0; tw < kBTW; ++tw) {
                    __builtin_amdgcn_s_setprio(1);      // matrix-product issue goes first, the other waves' vector work fills in behind
                    f32x4 na0 = zf, na1 = zf, ng0 = zf, ng1 = zf;
                    if (tw + 1 < kBTW) front(tw + 1, na0, na1, ng0, ng1);
                    if (tw > 0) back(tw - 1, pap, pdp);
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_s_setprio(0);
                    __builtin_amdgcn_sched_barrier(0);
                    float av[8], ds[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        av[e] = fast_exp2(a0[e]);
                        av[e + 4] = fast_exp2(a1[e]);
                        ds[e] = av[e] * fmaf(nea[e], de[tw], g0[e]);
                        ds[e + 4] = av[e + 4] * fmaf(neb[e], de[tw], g1[e]);
                    }
                    pap = pack8(av);
                    pdp = pack8(ds);
                    a0 = na0; a1 = na1; g0 = ng0; g1 = ng1;
                    __builtin_amdgcn_sched_barrier(0);
                }
                back(kBTW - 1, pap, pdp);
                continue;
            }
#pragma unroll
            for (int tw = 0; tw < kBTW; ++tw) {
                f32x4 a0 = la, a1 = lb, s0 = zf, s1 = zf, g10 = DROP ? zf : da, g11 = DROP ? zf : db, g20 = zf, g21 = zf;
                __builtin_amdgcn_s_setprio(1);      // matrix-product issue goes first, the other waves' vector work fills in behind
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) {
                    a0 = M_::mma(q0[kd], kb[tw][kd], a0);
                    a1 = M_::mma(q1[kd], kb[tw][kd], a1);
                    s0 = M_::mma(q0[kd], kb[tw][kd], s0);
                    s1 = M_::mma(q1[kd], kb[tw][kd], s1);
                    g10 = Pb::mma(d0[kd], vb[tw][kd], g10);
                    g11 = Pb::mma(d1[kd], vb[tw][kd], g11);
                    g20 = Pb::mma(z0[kd], yb[tw][kd], g20);
                    g21 = Pb::mma(z1[kd], yb[tw][kd], g21);
                }
                __builtin_amdgcn_s_setprio(0);
                float av[8], ds[8];
                if constexpr (DROP) {
                    const uint32_t n = (uint32_t)min(t0 + tw * 16 + c16, wg_n1 - 1);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const uint32_t m = (uint32_t)(a.m0 + 32 * ks + (e >> 2) * 16 + 4 * g + (e & 3));
                        const float k1 = dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 0u, (uint32_t)bh, m, n);
                        const float k2 = dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 1u, (uint32_t)bh, m, n);
                        const float wa = fast_exp2(e < 4 ? a0[e & 3] : a1[e & 3]);
                        const float g1 = e < 4 ? g10[e & 3] : g11[e & 3], g2 = e < 4 ? g20[e & 3] : g21[e & 3];
                        const float sc = e < 4 ? s0[e & 3] : s1[e & 3], dl = e < 4 ? da[e & 3] : db[e & 3];
                        ds[e] = wa * fmaf(k1, g1, dl) + fast_exp2(sc - r2[tw]) * (k2 * g2 - de[tw]);
                        av[e] = wa * k1;
                    }
                } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    av[e] = fast_exp2(a0[e]);
                    av[e + 4] = fast_exp2(a1[e]);
                    ds[e] = av[e] * g10[e] + fast_exp2(s0[e] - r2[tw]) * (g20[e] - de[tw]);
                    ds[e + 4] = av[e + 4] * g11[e] + fast_exp2(s1[e] - r2[tw]) * (g21[e] - de[tw]);
                }
                }
                const u32x4 pa = pack8(av), pd = pack8(ds);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    adv[tw][rt] = Pb::mma(odz[rt], pa, adv[tw][rt]);
                    adk[tw][rt] = Pb::mma(oq[rt], pd, adk[tw][rt]);
                }
            }
        }

        // lane (token c16, group g) owns d = (D/4) g .. (D/4) g + D/4 - 1 of both gradients
#pragma unroll
        for (int tw = 0; tw < kBTW; ++tw) {
            const int n = t0 + tw * 16 + c16;
            if (n >= wg_n1) continue;
            auto put = [&](uint16_t* base, int64_t stride, const f32x4 (&acc)[RT]) {
                uint16_t* p = base + (int64_t)n * stride + (D / 4) * g;
                uint32_t o[2 * RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    f32x4 t = acc[rt];
                    if (a.accumulate) {       // a later chunk of latents: add to what the earlier launches stored
                        const uint2 old = *reinterpret_cast<const uint2*>(p + 4 * rt);
                        t[0] += M_::unpack(uint16_t(old.x & 0xffffu));
                        t[1] += M_::unpack(uint16_t(old.x >> 16));
                        t[2] += M_::unpack(uint16_t(old.y & 0xffffu));
                        t[3] += M_::unpack(uint16_t(old.y >> 16));
                    }
                    o[2 * rt] = M_::pack2(t[0], t[1]);
                    o[2 * rt + 1] = M_::pack2(t[2], t[3]);
                }
                if constexpr (RT == 1) {
                    *reinterpret_cast<uint2*>(p) = make_uint2(o[0], o[1]);
                } else {
#pragma unroll
                    for (int i = 0; i < RT / 2; ++i)
                        *reinterpret_cast<u32x4*>(p + 8 * i) = u32x4{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
                }
            };
            put(dk, a.dks[2], adk[tw]);
            if (a.dv) put(dv, a.dvs[2], adv[tw]);
        }
    }
    };
    if constexpr (DROPK) {
        walk(std::false_type{}, std::true_type{}, 0.f);
    } else {
        if (fast) walk(std::true_type{}, std::false_type{}, lmax2);
        else walk(std::false_type{}, std::false_type{}, 0.f);
    }
}

template <typename T, int D, int MODE, bool DROPK>
hipError_t lat_launch(const MixerBwdArgs& a, hipStream_t st)
{
    // 4 latent tiles per wave need too many registers at D = 64 in the dq pass, and with the keep factors of a forward
    // with dropout everywhere (then 2 tiles, 1 at D = 64 in the dq pass)
    if (a.M % 256 == 0 && !(D == 64 && MODE == 1) && !DROPK) {
        hipLaunchKernelGGL((bwd_lat_kernel<T, D, DROPK ? 2 : 4, MODE, DROPK>), dim3(a.n_splits * (a.M / 256), a.H, a.B), dim3(256), 0, st, a);
    } else if (a.M % 128 == 0 && !(DROPK && D == 64 && MODE == 1)) {
        hipLaunchKernelGGL((bwd_lat_kernel<T, D, 2, MODE, DROPK>), dim3(a.n_splits * (a.M / 128), a.H, a.B), dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((bwd_lat_kernel<T, D, 1, MODE, DROPK>), dim3(a.n_splits * ((a.M + 63) / 64), a.H, a.B), dim3(256), 0, st, a);
    }
    return hipGetLastError();
}

template <typename T, int D, bool DROPK>
hipError_t bwd_all(const MixerBwdArgs& a, hipStream_t st)
{
    const int64_t lat = (int64_t)a.B * a.H * a.M;
    MixerBwdArgs a0 = a;          // the dz pass and its merge work in the dz pass's own split of the token axis
    a0.n_splits = a.n_splits0;
    a0.tokens_per_split = a.tokens_per_split0;
    // bf16 at D = 32 without dropout: the token-parallel passes on the 32x32x16 product.  The scatter half alone stays on
    // the two-exponential form, which only the 16x16x32 token and dq passes run at full speed.
    const bool mfma32 = !DROPK && !a.no_mfma32 && std::is_same<T, bf16_t>::value && bwd_dz32_supported(1, a.M, D);
    const bool dz32 = mfma32, dq32 = mfma32 && a.half != 2;
    hipError_t e = hipSuccess;
    if (a.half != 0) {
        if (DROPK) return hipErrorInvalidValue;
        const int64_t items = std::max<int64_t>((int64_t)a.B * a.H * (a.half == 1 ? a.N : a.M), lat);
        hipLaunchKernelGGL(bwd_half_prep_kernel, dim3((unsigned)std::min<int64_t>((items + 255) / 256, 4096)), dim3(256), 0, st, a);
    }
    if (a.half != 1) {      // the gather half is handed dz
        e = dz32 ? launch_bwd_dz32(a0, st) : lat_launch<T, D, 0, DROPK>(a0, st);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(bwd_merge_kernel<0>, dim3((unsigned)((lat * (D / 4) + 255) / 256)), dim3(256), 0, st, a0);
    }
    // the token pass on the 32x32x16 product takes the (b,h) of the unshifted one-exponential form; the kernel below
    // then only works on the others (normally none: its workgroups return at once)
    const bool tok32 = dq32 && bwd_tok32_supported(1, a.M, D);
    if (tok32) {
        e = launch_bwd_tok32(a, st);
        if (e != hipSuccess) return e;
    }
    {
        auto kern = bwd_tok_kernel<T, D, DROPK>;
        // the latents are covered in 1, 2 or 4 launches, each with the operand sets of its chunk in LDS
        const int chunks = mixer_bwd_tok_chunks(a.M, D);
        if (chunks == 0) return hipErrorInvalidValue;
        const int mc = a.M / chunks;
        // per-latent scalar tables behind the operand sets where the LDS has room
        const bool scal_lds = mixer_bwd_lds_bytes(mc, D) + (size_t)3 * mc * sizeof(float) <= 160 * 1024;
        const size_t lds = mixer_bwd_lds_bytes(mc, D) + (scal_lds ? (size_t)3 * mc * sizeof(float) : 0);
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        // one workgroup per compute unit, ranges a multiple of its 512-token pass
        const int64_t per_bh = (device_cus() + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H);
        int64_t tpw = (a.N + per_bh - 1) / per_bh;
        constexpr int pass = kTokWaves<D> * 16 * kTokTiles<D>;
        tpw = ((tpw + pass - 1) / pass) * pass;
        for (int c = 0; c < chunks; ++c) {
            MixerBwdArgs ac = a;
            ac.m0 = c * mc;
            ac.mc = mc;
            ac.accumulate = c > 0;
            ac.scal_lds = scal_lds ? 1 : 0;
            ac.only_form = tok32 ? 2 : 0;
            hipLaunchKernelGGL(kern, dim3((unsigned)((a.N + tpw - 1) / tpw), a.H, a.B), dim3(64 * kTokWaves<D>), lds, st, ac, (int)tpw);
        }
    }
    e = dq32 ? launch_bwd_dq32(a, st) : lat_launch<T, D, 1, DROPK>(a, st);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(bwd_merge_kernel<1>, dim3((unsigned)((lat * (D / 4) + 255) / 256)), dim3(256), 0, st, a);
    return hipGetLastError();
}

template <typename T>
hipError_t bwd_d(const MixerBwdArgs& a, hipStream_t st)
{
    if (a.drop_thr != 0) {      // the forward dropped weights: kernels that regenerate the keep masks
        switch (a.D) {
            case 16: return bwd_all<T, 16, true>(a, st);
            case 32: return bwd_all<T, 32, true>(a, st);
            case 64: return bwd_all<T, 64, true>(a, st);
            default: return hipErrorInvalidValue;
        }
    }
    switch (a.D) {
        case 16: return bwd_all<T, 16, false>(a, st);
        case 32: return bwd_all<T, 32, false>(a, st);
        case 64: return bwd_all<T, 64, false>(a, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

size_t mixer_bwd_lds_bytes(int M, int D) { return (size_t)M * D * 2 * 5; }

// Launches of the token-side kernel needed to cover M latents (each takes a chunk that is a multiple of 32 and whose
// five operand sets fit the 160 KB of LDS), or 0 when even four do not do.
int mixer_bwd_tok_chunks(int M, int D)
{
    for (int c = 1; c <= 4; c *= 2)
        if (M % (32 * c) == 0 && mixer_bwd_lds_bytes(M / c, D) <= 160 * 1024) return c;
    return 0;
}

bool mixer_bwd_supported(int dtype, int M, int D)
{
    return (dtype == 1 || dtype == 2) && (D == 16 || D == 32 || D == 64) && M >= 32 && M % 32 == 0 &&
           mixer_bwd_tok_chunks(M, D) > 0;
}

hipError_t launch_mixer_bwd(const MixerBwdArgs& a, int dtype, hipStream_t st)
{
    return dtype == 1 ? bwd_d<bf16_t>(a, st) : bwd_d<f16_t>(a, st);
}

}  // namespace flare
