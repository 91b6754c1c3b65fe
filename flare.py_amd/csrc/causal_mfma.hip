// Causal FLARE chunked prefill on the matrix cores (bf16 / f16, D in {32, 64}, M in {128, 256}).
//
// Same definition and state as causal.hip:  z_t = gather over tokens <= t,  y_t = scatter of z_t.
// One workgroup (4 waves) owns one (b,h) and walks its tokens in blocks of 16; wave w owns
// MW = M/4 latents (their scores, running denominators and state rows), so the only cross-wave
// step is the sum over latents of the 16 x D output tile, done through LDS with one barrier per
// block.  Per block and wave, with P = exp2(score - mu0) for the wave's latents (mu0 = the shift
// of the incoming state, 0 for a fresh one; no running maximum):
//   dcum[t,m] = den[m] + sum_{tau<=t} P[tau,m]          (MFMA with a lower-triangular ones matrix)
//   W[t,m]    = P[t,m] f[m],  f[m] = exp2(mu0[m] - max_m mu0)     (the token's softmax weight over the latents:
//                                                                   one shift for all latents; f = 1 unless
//                                                                   the state carries per-latent shifts)
//   G[t,m]    = W[t,m] / dcum[t,m]
//   Y[t,:]   += G[t,:] U  +  tril(G P^T)[t,:] V          (U = state numerator [m,d])
//   r[t]     += sum_m W[t,m]                             (MFMA against the factors f)
//   U[m,:]   += P[:,m]^T V ;  den[m] += sum_tau P[tau,m]
// and finally y_t = (sum over waves of Y[t,:]) / (sum over waves of r[t]).
// A 16x16 accumulator tile (lane = column c16, registers = rows 4g..4g+3) is reused directly as the
// A or B operand of a 16x16x16 MFMA whose contraction runs over those rows; operands that need the
// other orientation (tokens in lanes, latents in registers) go through a wave-private LDS tile and
// the transpose read.  Working without a running maximum is validated (finite outputs, softmax
// sums and denominators inside 2^-60..2^120); a (b,h) that fails leaves its state untouched and
// raises a flag, and the fp32 kernel of causal.hip, launched right after, redoes exactly those.
#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLMin = 8.6736174e-19f, kLMax = 1.329228e36f;   // 2^-60, 2^120

template <typename T> struct Mm;
template <> struct Mm<bf16_t> {
    static constexpr uint32_t kOnes2 = 0x3f803f80u;
    static __device__ __forceinline__ f32x4 mma32(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mma16(uint2 a, uint2 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float unpack(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
};
template <> struct Mm<f16_t> {
    static constexpr uint32_t kOnes2 = 0x3c003c00u;
    static __device__ __forceinline__ f32x4 mma32(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mma16(uint2 a, uint2 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float unpack(uint16_t b) { return float(__builtin_bit_cast(_Float16, b)); }
};

__device__ __forceinline__ uint2 tr16(const void* lds_addr)
{
    // The pointer reaches the intrinsic through an integer cast, so the compiler may not see that it
    // aliases the ordinary stores that fill the tile: keep it from moving either across the read.
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    asm volatile("" ::: "memory");
    const s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)lds_addr);
    asm volatile("" ::: "memory");
    return __builtin_bit_cast(uint2, r);
}

// The same read at a byte address in LDS plus a compile-time offset: the offset goes into the instruction's offset
// field, so the many reads of one step share a few address registers (as pointers each would occupy its own).
template <int OFF>
__device__ __forceinline__ uint2 tr16_at(uint32_t lds_byte_addr)
{
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    asm volatile("" ::: "memory");
    const s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)(lds_byte_addr + OFF));
    asm volatile("" ::: "memory");
    return __builtin_bit_cast(uint2, r);
}

// f(integral_constant<int, I>) for I = 0 .. N - 1, unrolled at compile time
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

typedef uint32_t u32v2 __attribute__((ext_vector_type(2)));
// An ordinary LDS read of a V (a scalar or a compiler vector type) at a byte address plus a compile-time offset (same reason).
template <typename V, int OFF>
__device__ __forceinline__ V lds_at(uint32_t lds_byte_addr)
{
    typedef const V __attribute__((address_space(3))) * ptr_t;
    return *(ptr_t)(uintptr_t)(lds_byte_addr + OFF);
}
// Keeps the compiler from folding an address into the expressions that use it (it would re-derive one register per use).
__device__ __forceinline__ uint32_t opaque(uint32_t x)
{
    asm volatile("" : "+v"(x));
    return x;
}

// The state's numerators and denominators are relative to a shift mu0[m] per latent, which cancels in
// z = U/den.  The softmax over the latents of one token's scores needs ONE shift for all latents
// instead: its weights are exp2(score - cref) = P[t,m] * exp2(mu0[m] - cref) with
// cref = max_m mu0[m].  For a state this kernel produced itself mu0 is the same for every latent and
// the factor is exactly 1; a state that comes from the fp32 kernel carries per-latent running maxima.
__device__ __forceinline__ float common_shift(const float* mu_g, int M, int lane)
{
    float mx = kNegBig;
    for (int m = lane; m < M; m += 256) {          // up to four loads in flight (M <= 256: one round trip)
        float mu[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) mu[u] = mu_g[m + 64 * u < M ? m + 64 * u : m];
#pragma unroll
        for (int u = 0; u < 4; ++u) mx = fmaxf(mx, mu[u] <= kNegBig ? 0.f : mu[u] * kLog2e);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    return mx;
}

constexpr int kTB = 16;   // tokens per block
constexpr int kVPad = 16; // elements of padding per V row in LDS (row stride D*2 + 32 bytes)

// STATE_ONLY = false: the full recurrence over the workgroup's token segment, from the incoming
// state plus the local states of all earlier segments (summed in segment order).  A single
// segment writes the state back itself; with several, the last one stages it in the workspace.
// STATE_ONLY = true: only the segment's local denominators and numerators (first phase).
template <typename T, int D, int KM, bool STATE_ONLY>
__global__ __launch_bounds__(256, 2) void causal_mfma_kernel(CausalArgs a, int step)
{
    constexpr int KD = D / 32;          // k-steps over d of the score product
    constexpr int DT = D / 16;          // 16-column tiles of d
    constexpr int CT = 2 * KM;          // 16-latent column tiles per wave
    constexpr int MW = 32 * KM;         // latents per wave
    constexpr int M = 4 * MW;
    constexpr int YS = D + 4;           // padded row stride (floats) of the output partials
    using M_ = Mm<T>;         // score product and output, in the element type of q, k, y
    using P_ = Mm<bf16_t>;    // every other product: probabilities, weights, state and values as bf16

    // V block, row-major; rows padded so that the transpose reads of 8 rows hit 8 different bank groups
    __shared__ __attribute__((aligned(16))) uint16_t vs[2][kTB][D + kVPad];
    __shared__ __attribute__((aligned(16))) uint16_t pt[4][MW][kTB];      // P^T per wave  [latent][token]
    __shared__ __attribute__((aligned(16))) uint16_t gt[4][MW][kTB];      // G^T per wave
    __shared__ __attribute__((aligned(16))) float yp[2][4][kTB][YS];      // output partials per wave
    __shared__ float rp[2][4][kTB];                                       // softmax-sum partials per wave
    __shared__ int bad_flag;

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H, seg = blockIdx.y;
    // this segment: tokens n_lo .. N-1 (the first phase walks the parts of its piece instead, see below)
    int n_lo = seg * a.seg_len, N = min(a.N, n_lo + a.seg_len);
    const bool single = a.n_segs == 1;
    float* seg_den = a.seg_den + ((int64_t)bh * a.n_slots + a.n_slots - 1) * M;        // staging slot of the final state
    float* seg_num = a.seg_num + ((int64_t)bh * a.n_slots + a.n_slots - 1) * M * D;
    const int n_before = STATE_ONLY ? 0 : causal_slots_before(seg, a.seg_len, a.piece_len);
    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    uint16_t* y = (uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    float* mu_g = a.mu + (int64_t)bh * M;
    float* den_g = a.den + (int64_t)bh * M;
    float* num_g = a.num + (int64_t)bh * M * D;
    const float sl2 = a.scale * kLog2e;
    const int m0 = w * MW;

    if (tid == 0) bad_flag = 0;

    // latent operands (B of the score product), log2-scaled; shift and denominators per column
    u32x4 qb[CT][KD];
    f32x4 negmu[CT], den[CT];
    float mu0[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = m0 + ct * 16 + c16;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const u32x4 raw = *reinterpret_cast<const u32x4*>(q + (int64_t)m * a.qs[2] + kd * 32 + g * 8);
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o[i] = M_::pack2(M_::unpack(uint16_t(raw[i] & 0xffffu)) * sl2, M_::unpack(uint16_t(raw[i] >> 16)) * sl2);
            qb[ct][kd] = o;
        }
        const float mu = mu_g[m];
        mu0[ct] = mu <= kNegBig ? 0.f : mu * kLog2e;
        negmu[ct] = f32x4{-mu0[ct], -mu0[ct], -mu0[ct], -mu0[ct]};
        float d0 = 0.f;
        if constexpr (!STATE_ONLY) {
            const float dn_in = den_g[m];          // read whether the latent is fresh or not (no load behind a wait for mu)
            d0 = mu <= kNegBig ? 0.f : dn_in;
        }
        if (!STATE_ONLY)
            for (int s = 0; s < n_before; ++s) d0 += a.seg_den[((int64_t)bh * a.n_slots + s) * M + m];
        den[ct] = f32x4{d0, d0, d0, d0};
    }
    // state numerator U[m, d]: tile (mt, dt) holds rows m0 + 16 mt + 4g + r, column 16 dt + c16
    f32x4 U[CT][DT];
#pragma unroll
    for (int mt = 0; mt < CT; ++mt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + mt * 16 + 4 * g + r;
                float u = 0.f;
                if constexpr (!STATE_ONLY) {
                    const float mu_m = mu_g[m], un = num_g[(int64_t)m * D + dt * 16 + c16];
                    u = mu_m <= kNegBig ? 0.f : un;
                }
                if (!STATE_ONLY)
                    for (int s = 0; s < n_before; ++s)
                        u += a.seg_num[(((int64_t)bh * a.n_slots + s) * M + m) * D + dt * 16 + c16];
                U[mt][dt][r] = u;
            }

    // constant operands: lower-triangular ones L[t = c16][tau = 4g + e] and all ones
    uint2 ltri, ones4 = make_uint2(P_::kOnes2, P_::kOnes2);
    {
        const uint32_t one = P_::kOnes2 & 0xffffu;
        uint32_t e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = (4 * g + i <= c16) ? one : 0u;
        ltri = make_uint2(e[0] | (e[1] << 16), e[2] | (e[3] << 16));
    }
    // weights of the softmax over latents: fw[ct] = exp2(mu0 - cref) per column, and the same factors as a B
    // operand (k-slots = the wave's latents 32 km + 4g + e / 32 km + 16 + 4g + e - 4) for the row sums
    const float cref = common_shift(mu_g, M, lane);
    float fw[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) fw[ct] = fast_exp2(mu0[ct] - cref);
    u32x4 fop[KM];
#pragma unroll
    for (int km = 0; km < KM; ++km) {
        float f8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float mu = mu_g[m0 + km * 32 + (e >> 2) * 16 + 4 * g + (e & 3)];
            f8[e] = fast_exp2((mu <= kNegBig ? 0.f : mu * kLog2e) - cref);
        }
        fop[km] = u32x4{P_::pack2(f8[0], f8[1]), P_::pack2(f8[2], f8[3]), P_::pack2(f8[4], f8[5]), P_::pack2(f8[6], f8[7])};
    }

    // block staging: K as A operand straight from global memory, V through LDS (threads < 2 D)
    u32x4 ka[KD], kn[KD], vr;
    auto load_block = [&](int n0, u32x4 (&kd_)[KD]) {
        const int n = min(n0 + c16, N - 1);
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) kd_[kd] = *reinterpret_cast<const u32x4*>(k + (int64_t)n * a.ks[2] + kd * 32 + g * 8);
        if (tid < 2 * D) {
            const int tok = tid / (D / 8), ch = tid % (D / 8);
            vr = *reinterpret_cast<const u32x4*>(v + (int64_t)min(n0 + tok, N - 1) * a.vs[2] + ch * 8);
        }
    };
    auto store_v = [&](int buf) {
        if (tid < 2 * D) {
            const int tok = tid / (D / 8), ch = tid % (D / 8);
            u32x4 o = vr;
            if constexpr (!std::is_same<T, bf16_t>::value) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    o[i] = P_::pack2(M_::unpack(uint16_t(vr[i] & 0xffffu)), M_::unpack(uint16_t(vr[i] >> 16)));
            }
            *reinterpret_cast<u32x4*>(&vs[buf][tok][ch * 8]) = o;
        }
    };

    if constexpr (STATE_ONLY) {
        // The first phase never raises a flag, and the recurrence phase starts after it has finished: its first
        // workgroup clears the (b,h)'s redo flag (by a kernel, so that a caller may capture the call in a graph).
        if (seg == 0 && tid == 0) a.flags[bh] = 0;
        // Local states of this workgroup's piece of the tokens: one per segment the piece reaches into (n_lo, N are
        // set to each such part in turn).  A 16-token block is too little work here to cover the memory
        // latency of its own prefetch, so this phase walks 64-token tiles: K as four A operands per
        // lane, V through a 64-row LDS tile.  Three register sets take turns, each refilled with the tile
        // three ahead as soon as its own has been used: loads are unconditional (rows past the end of
        // the segment repeat its last row) and never copied between registers, so that every wait counts
        // exactly what is in flight.
        // K and V tiles in LDS (K rows padded by 8 elements: the 16 rows a wave reads as one operand then start in 16
        // different bank groups; V rows by kVPad for the transposing reads)
        constexpr int KROW = (D + 8) * 2, VROW = (D + kVPad) * 2;       // row strides in bytes
        __shared__ __attribute__((aligned(16))) uint8_t k64[2][64 * KROW];
        __shared__ __attribute__((aligned(16))) uint8_t v64[2][64 * VROW];
        constexpr int VPT = 64 * (D / 8) / 256;     // 16-byte K and V chunks per thread and tile
        static_assert(64 * (D / 8) == VPT * 256, "every thread stages the same number of chunks");
        struct Tile { u32x4 k[VPT]; u32x4 v[VPT]; };
        auto fetch = [&](int n0, Tile& t) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const int c = tid + i * 256, tok = c / (D / 8), ch = c % (D / 8);
                const int64_t row = min(n0 + tok, N - 1);
                t.k[i] = *reinterpret_cast<const u32x4*>(k + row * a.ks[2] + ch * 8);
                t.v[i] = *reinterpret_cast<const u32x4*>(v + row * a.vs[2] + ch * 8);
            }
        };
        // V rows of absent tokens are staged as zeros (their probabilities then add nothing to the numerators)
        auto stage = [&](int n0, int buf, const Tile& t) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const int c = tid + i * 256, tok = c / (D / 8), ch = c % (D / 8);
                u32x4 o = t.v[i];
                if constexpr (!std::is_same<T, bf16_t>::value) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[j] = P_::pack2(M_::unpack(uint16_t(t.v[i][j] & 0xffffu)), M_::unpack(uint16_t(t.v[i][j] >> 16)));
                }
                if (n0 + tok >= N) o = u32x4{0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4*>(&k64[buf][tok * KROW + ch * 16]) = t.k[i];
                *reinterpret_cast<u32x4*>(&v64[buf][tok * VROW + ch * 16]) = o;
            }
        };
        // byte addresses in LDS of the lane's pieces: K row c16, 16 bytes at 8g elements; V row 4g + (c16 >> 2), piece c16 & 3
        const uint32_t k_b = opaque((uint32_t)(uintptr_t)&k64[0][0] + c16 * KROW + g * 16);
        const uint32_t v_b = opaque((uint32_t)(uintptr_t)&v64[0][0] + (4 * g + (c16 >> 2)) * VROW + (c16 & 3) * 8);
        // the tile's contribution, two 16-token blocks per product (k-slots 8g + i: token 4g + i of the first block,
        // 8g + 4 + i: of the second); the denominators count live tokens only (the A operand of their product holds
        // ones in the k-slots of live tokens)
        auto work = [&](int n0, auto buf_c) __attribute__((always_inline)) {
            constexpr int KB = decltype(buf_c)::value * 64 * KROW, VB = decltype(buf_c)::value * 64 * VROW;
            static_for<2>([&](auto sp_c) {
                constexpr int sp = decltype(sp_c)::value;
                const int tb = N - (n0 + sp * 32);   // tokens >= tb of this pair of blocks are beyond the part
                u32x4 live8 = u32x4{ones4.x, ones4.y, ones4.x, ones4.y};
                if (tb < 32) {
                    const uint32_t one = P_::kOnes2 & 0xffffu;
#pragma unroll
                    for (int hb = 0; hb < 2; ++hb) {
                        const int t0 = hb * 16 + 4 * g;
                        live8[2 * hb] = (t0 + 0 < tb ? one : 0u) | (t0 + 1 < tb ? one << 16 : 0u);
                        live8[2 * hb + 1] = (t0 + 2 < tb ? one : 0u) | (t0 + 3 < tb ? one << 16 : 0u);
                    }
                }
                // all operands of the pair of blocks requested at once
                u32x4 ka[2][KD], vop[DT];
                static_for<KD>([&](auto kd_c) {
                    constexpr int kd = decltype(kd_c)::value;
                    ka[0][kd] = lds_at<u32x4, KB + (2 * sp) * 16 * KROW + kd * 64>(k_b);
                    ka[1][kd] = lds_at<u32x4, KB + (2 * sp + 1) * 16 * KROW + kd * 64>(k_b);
                });
                static_for<DT>([&](auto dt_c) {
                    constexpr int dt = decltype(dt_c)::value;
                    const uint2 lo = tr16_at<VB + sp * 32 * VROW + dt * 32>(v_b);
                    const uint2 hi = tr16_at<VB + (sp * 32 + 16) * VROW + dt * 32>(v_b);
                    vop[dt] = u32x4{lo.x, lo.y, hi.x, hi.y};
                });
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    f32x4 s0 = negmu[ct], s1 = negmu[ct];
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd) {
                        s0 = M_::mma32(ka[0][kd], qb[ct][kd], s0);
                        s1 = M_::mma32(ka[1][kd], qb[ct][kd], s1);
                    }
                    const u32x4 ppk = u32x4{P_::pack2(fast_exp2(s0[0]), fast_exp2(s0[1])), P_::pack2(fast_exp2(s0[2]), fast_exp2(s0[3])),
                                            P_::pack2(fast_exp2(s1[0]), fast_exp2(s1[1])), P_::pack2(fast_exp2(s1[2]), fast_exp2(s1[3]))};
                    den[ct] = P_::mma32(live8, ppk, den[ct]);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) U[ct][dt] = P_::mma32(ppk, vop[dt], U[ct][dt]);
                }
            });
        };
        const int p_lo = seg * a.piece_len, p_hi = min(p_lo + a.piece_len, (a.n_segs - 1) * a.seg_len);
        for (int s = p_lo / a.seg_len; s <= (p_hi - 1) / a.seg_len; ++s) {
        n_lo = max(p_lo, s * a.seg_len);
        N = min(p_hi, (s + 1) * a.seg_len);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            den[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) U[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        __syncthreads();   // the part before has read its last tile
        // Two register sets take turns: each is staged into LDS one tile ahead of its use and refilled at once with the
        // tile two further on.  Loads are unconditional (rows past the end of the part repeat its last row) and never
        // copied between registers, so that every wait counts exactly what is in flight.
        Tile ta, tb_;
        fetch(n_lo, ta);
        fetch(n_lo + 64, tb_);
        stage(n_lo, 0, ta);
        fetch(n_lo + 128, ta);
        __syncthreads();
        // Whole pairs of tiles in a loop with one exit at its bottom, a last odd tile behind it: an exit from the middle
        // of the pair would reach the loop's head again in the compiler's control flow, and with prefetches in flight on
        // that path every pass through the head would wait for all of them.
        const int tiles = (N - n_lo + 63) >> 6;
        int n0 = n_lo;
        for (int gi = 0; gi < tiles / 2; ++gi, n0 += 128) {
            // tile n0 (in buffer 0); the next tile goes into buffer 1 meanwhile
            work(n0, std::integral_constant<int, 0>{});
            stage(n0 + 64, 1, tb_);
            fetch(n0 + 192, tb_);
            __syncthreads();
            work(n0 + 64, std::integral_constant<int, 1>{});
            stage(n0 + 128, 0, ta);
            fetch(n0 + 256, ta);
            __syncthreads();
        }
        if (tiles & 1) work(n0, std::integral_constant<int, 0>{});
        // nothing of this part stays in flight (the prefetches past its end were never used)
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        // local state of the part, relative to the shift of the incoming state; whatever
        // overflowed or vanished here is caught by the checks of the segments that use it
        const int64_t slot = (int64_t)bh * a.n_slots + causal_slot(seg, s, a.seg_len, a.piece_len);
        float* part_den = a.seg_den + slot * M;
        float* part_num = a.seg_num + slot * M * D;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (g == 0) part_den[m0 + ct * 16 + c16] = den[ct][0];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) part_num[(int64_t)(m0 + ct * 16 + 4 * g + r) * D + dt * 16 + c16] = U[ct][dt][r];
        }
        }
        return;
    }

    bool bad = false;
    load_block(n_lo, ka);
    store_v(0);
    if (n_lo + step < N) load_block(n_lo + step, kn);
    __syncthreads();

    int it = 0;
    // step = 16: chunked prefill; step = 1: recurrent decode, one token per block (rows >= tb are masked)
    for (int n0 = n_lo; n0 < N; n0 += step, ++it) {
        const int buf = it & 1;
        const int tb = min(step, N - n0);

        // scores and probabilities of the wave's latents: rows tau = 4g + r, column m = c16
        float p[CT][4];
        uint2 ppk[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f32x4 s = negmu[ct];
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) s = M_::mma32(ka[kd], qb[ct][kd], s);
#pragma unroll
            for (int r = 0; r < 4; ++r) p[ct][r] = (4 * g + r < tb) ? fast_exp2(s[r]) : 0.f;
            ppk[ct] = make_uint2(P_::pack2(p[ct][0], p[ct][1]), P_::pack2(p[ct][2], p[ct][3]));
        }
        // running denominators: dcum = den + L P ; den += 1 P ; G = P / dcum
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const f32x4 dc = P_::mma16(ltri, ppk[ct], den[ct]);
            den[ct] = P_::mma16(ones4, ppk[ct], den[ct]);
            float gv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) gv[r] = p[ct][r] > 0.f ? p[ct][r] * fw[ct] * __builtin_amdgcn_rcpf(dc[r]) : 0.f;
            const uint2 gpk = make_uint2(P_::pack2(gv[0], gv[1]), P_::pack2(gv[2], gv[3]));
            *reinterpret_cast<uint2*>(&pt[w][ct * 16 + c16][4 * g]) = ppk[ct];
            *reinterpret_cast<uint2*>(&gt[w][ct * 16 + c16][4 * g]) = gpk;
        }
        // operands with tokens in lanes and latents in k-slots (e < 4: tile 2 km, e >= 4: tile 2 km + 1)
        u32x4 pop[KM], gop[KM];
#pragma unroll
        for (int km = 0; km < KM; ++km) {
            const int r0 = km * 32 + 4 * g + (c16 >> 2), r1 = r0 + 16, piece = (c16 & 3) * 4;
            const uint2 p0 = tr16(&pt[w][r0][piece]), p1 = tr16(&pt[w][r1][piece]);
            const uint2 g0 = tr16(&gt[w][r0][piece]), g1 = tr16(&gt[w][r1][piece]);
            pop[km] = u32x4{p0.x, p0.y, p1.x, p1.y};
            gop[km] = u32x4{g0.x, g0.y, g1.x, g1.y};
        }
        // V operand (k-slots = tokens 4g..4g+3, lane = column d)
        uint2 vop[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vop[dt] = tr16(&vs[buf][4 * g + (c16 >> 2)][dt * 16 + (c16 & 3) * 4]);

        // intra-block matrix AccT[tau, t] = sum_m P[tau,m] G[t,m], masked to tau <= t, and r[t]
        f32x4 acct = {0.f, 0.f, 0.f, 0.f}, rsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int km = 0; km < KM; ++km) {
            acct = P_::mma32(pop[km], gop[km], acct);
            rsum = P_::mma32(pop[km], fop[km], rsum);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) acct[r] = (4 * g + r <= c16) ? acct[r] : 0.f;
        const uint2 aop = make_uint2(P_::pack2(acct[0], acct[1]), P_::pack2(acct[2], acct[3]));

        // output partial over the wave's latents, then the state update
        f32x4 yacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int km = 0; km < KM; ++km) {
                const f32x4 u0 = U[2 * km][dt], u1 = U[2 * km + 1][dt];
                const u32x4 ub = {P_::pack2(u0[0], u0[1]), P_::pack2(u0[2], u0[3]),
                                  P_::pack2(u1[0], u1[1]), P_::pack2(u1[2], u1[3])};
                acc = P_::mma32(gop[km], ub, acc);
            }
            yacc[dt] = P_::mma16(aop, vop[dt], acc);
        }
#pragma unroll
        for (int mt = 0; mt < CT; ++mt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) U[mt][dt] = P_::mma16(ppk[mt], vop[dt], U[mt][dt]);

        // partials to LDS (rows t = 4g + r, column d = 16 dt + c16)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) yp[buf][w][4 * g + r][dt * 16 + c16] = yacc[dt][r];
        if (c16 == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) rp[buf][w][4 * g + r] = rsum[r];
        }

        // stage the next block
        if (n0 + step < N) {
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) ka[kd] = kn[kd];
            store_v(buf ^ 1);
            if (n0 + 2 * step < N) load_block(n0 + 2 * step, kn);
        }
        __syncthreads();

        // y[t, :] = sum_w Y_w[t, :] / sum_w r_w[t]; thread = (token, 4 consecutive d)
        for (int idx = tid; idx < kTB * (D / 4); idx += 256) {
            const int t = idx / (D / 4), d4 = (idx % (D / 4)) * 4;
            const f32x4 s = *reinterpret_cast<const f32x4*>(&yp[buf][0][t][d4]) + *reinterpret_cast<const f32x4*>(&yp[buf][1][t][d4]) +
                            *reinterpret_cast<const f32x4*>(&yp[buf][2][t][d4]) + *reinterpret_cast<const f32x4*>(&yp[buf][3][t][d4]);
            const float r = rp[buf][0][t] + rp[buf][1][t] + rp[buf][2][t] + rp[buf][3][t];
            if (t < tb) {
                const float inv = 1.f / r;
                const f32x4 o = s * inv;
                bad = bad || !(r >= kLMin && r <= kLMax) || !(fabsf(o[0]) + fabsf(o[1]) + fabsf(o[2]) + fabsf(o[3]) <= 3.0e38f);
                *reinterpret_cast<uint2*>(y + (int64_t)(n0 + t) * a.ys[2] + d4) =
                    make_uint2(M_::pack2(o[0], o[1]), M_::pack2(o[2], o[3]));
                if (a.lse && d4 == 0) a.lse[(int64_t)bh * a.N + n0 + t] = (cref + __log2f(r)) * kLn2;
            }
        }
    }

    // validate the final denominators, then publish the state (or the redo flag).  With several
    // segments the flags were cleared beforehand and are only ever raised; the last segment
    // stages the state in its workspace slot and a commit kernel copies it once every segment
    // of the (b,h) has passed.
    const bool last = seg == a.n_segs - 1;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) bad = bad || (last && !(den[ct][0] >= kLMin && den[ct][0] <= kLMax));
    if (__any(bad) && lane == 0) bad_flag = 1;
    __syncthreads();
    if (bad_flag) {
        if (tid == 0) a.flags[bh] = 1;
        return;
    }
    if (single && tid == 0) a.flags[bh] = 0;
    if (!last) return;
    float* den_o = single ? den_g : seg_den;
    float* num_o = single ? num_g : seg_num;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = m0 + ct * 16 + c16;
        if (g == 0) {
            if (single) mu_g[m] = mu0[ct] * kLn2;
            den_o[m] = den[ct][0];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) num_o[(int64_t)(m0 + ct * 16 + 4 * g + r) * D + dt * 16 + c16] = U[ct][dt][r];
    }
}

// ---- 64-token chunks, tokens split across the waves (M = 128) ---------------------------------
// The full recurrence again, organised the other way round: a chunk of 64 tokens per step, wave w
// owning tokens 16w..16w+15 of the chunk for everything on the token side (all 128 latents: scores,
// P, running denominators, G, the output rows) and latents 32w..32w+31 for the state update.  The
// output rows need no sum across waves any more, and one chunk costs two barriers instead of four
// blocks with a dependent chain and a barrier each.  Per chunk, P = exp2(score - mu0) as above:
//   cs_w[m]   = sum over the wave's tokens of P                      (published with P^T in LDS)
//   dcum[t,m] = den[m] + sum_{w' < w} cs_w'[m] + (L P_w)[t,m]
//   G = P / dcum;   Y_w = G U0 + sum_{w' <= w} tril?(G P_w'^T) V_w'    (tril on the diagonal tile only)
//   U[own m] += sum_w' P_w'[:, m]^T V_w';   den += sum_w' cs_w'
// U0 = the state at the start of the chunk, published by its owners as bf16 B operands in LDS.
constexpr int kChunk = 64;
#define FLARE_CHUNK_FENCE() __builtin_amdgcn_sched_barrier(0)

template <int D> constexpr size_t causal_chunk_lds()
{
    // q operands, V chunk, P^T and G^T of the four waves, U0 operands, column sums
    return (size_t)8 * (D / 32) * 64 * 16 + (size_t)kChunk * (D + kVPad) * 2 + 2 * (size_t)4 * 128 * 16 * 2 +
           (size_t)4 * (D / 16) * 64 * 16 + (size_t)4 * 128 * 4 + (size_t)4 * 4 * 16 + (size_t)2 * 128 * 4;
}

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void causal_chunk_kernel(CausalArgs a)
{
    constexpr int M = 128, KD = D / 32, DT = D / 16, CTA = M / 16, KS = M / 32, MT = 2;
    constexpr int VPT = (kChunk * (D / 8) + 255) / 256;     // 16-byte V pieces per thread and chunk
    constexpr int VS = D + kVPad;                           // V row stride in LDS (elements)
    using M_ = Mm<T>;
    using P_ = Mm<bf16_t>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    u32x4* qs = reinterpret_cast<u32x4*>(smem);                                   // [CTA][KD][64]
    uint16_t* vs = reinterpret_cast<uint16_t*>(qs + CTA * KD * 64);               // [64][VS], VS = D + padding
    uint16_t* pt = vs + kChunk * VS;                                              // [4][M][16]
    uint16_t* gt = pt + 4 * M * 16;                                               // [4][M][16]
    u32x4* u0s = reinterpret_cast<u32x4*>(gt + 4 * M * 16);                       // [KS][DT][64]
    float* cs = reinterpret_cast<float*>(u0s + KS * DT * 64);                     // [M][4]: column sums of the four waves' P
    u32x4* fops = reinterpret_cast<u32x4*>(cs + 4 * M);                           // [KS][4]: weight factors as B operands
    float* mu0s = reinterpret_cast<float*>(fops + KS * 4);                        // [M] shift of each latent (log2 units)
    float* fws = mu0s + M;                                                        // [M] weight factor exp2(mu0 - cref)
    __shared__ int bad_flag;

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // uniform over the wave: the branches on it are scalar
    // The later waves of a chunk have more tiles of earlier tokens to go through and reach the barriers last: where two
    // waves of a SIMD compete for issue, they go first (measured: 1 % of the kernel).
    if (w == 3) __builtin_amdgcn_s_setprio(2); else if (w == 2) __builtin_amdgcn_s_setprio(1);
    const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H, seg = blockIdx.y;
    const int n_lo = seg * a.seg_len, N = min(a.N, n_lo + a.seg_len);
    const bool single = a.n_segs == 1;
    float* seg_den = a.seg_den + ((int64_t)bh * a.n_slots + a.n_slots - 1) * M;        // staging slot of the final state
    float* seg_num = a.seg_num + ((int64_t)bh * a.n_slots + a.n_slots - 1) * M * D;
    const int n_before = causal_slots_before(seg, a.seg_len, a.piece_len);
    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    uint16_t* y = (uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    float* mu_g = a.mu + (int64_t)bh * M;
    float* den_g = a.den + (int64_t)bh * M;
    float* num_g = a.num + (int64_t)bh * M * D;
    const float sl2 = a.scale * kLog2e;
    const int m0 = w * 32;
    uint16_t* ptw = pt + w * M * 16;      // this wave's P^T  [latent][token]
    uint16_t* gtw = gt + w * M * 16;      // this wave's G^T, later its output transposition tiles

    if (tid == 0) bad_flag = 0;

    // q as B operands of the score product (log2-scaled), for every latent tile
    for (int idx = tid; idx < CTA * KD * 64; idx += 256) {
        const int ln = idx & 63, kd = (idx >> 6) % KD, ct = idx / (64 * KD);
        const int m = ct * 16 + (ln & 15);
        const u32x4 raw = *reinterpret_cast<const u32x4*>(q + (int64_t)m * a.qs[2] + kd * 32 + (ln >> 4) * 8);
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            o[i] = M_::pack2(M_::unpack(uint16_t(raw[i] & 0xffffu)) * sl2, M_::unpack(uint16_t(raw[i] >> 16)) * sl2);
        qs[idx] = o;
    }
    // factors exp2(mu0 - cref) of the softmax over latents as B operands: k-step ks, lane group gg hold the
    // latents 32 ks + 4 gg + e (e < 4) and 32 ks + 16 + 4 gg + e - 4
    const float cref = common_shift(mu_g, M, lane);
    if (tid < KS * 4) {
        const int ks = tid >> 2, gg = tid & 3;
        float f8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float mu = mu_g[ks * 32 + (e >> 2) * 16 + 4 * gg + (e & 3)];
            f8[e] = fast_exp2((mu <= kNegBig ? 0.f : mu * kLog2e) - cref);
        }
        fops[tid] = u32x4{P_::pack2(f8[0], f8[1]), P_::pack2(f8[2], f8[3]), P_::pack2(f8[4], f8[5]), P_::pack2(f8[6], f8[7])};
    }
    // per-latent shift and weight factor: small tables in LDS (registers are short in this kernel)
    if (tid < M) {
        const float mu = mu_g[tid];
        const float m2 = mu <= kNegBig ? 0.f : mu * kLog2e;
        mu0s[tid] = m2;
        fws[tid] = fast_exp2(m2 - cref);
    }
    // running denominators of every latent (column c16 of tile ct), replicated in the waves
    // (the earlier segments' local states are added segment by segment, in segment order: every load of one
    // segment's contribution is issued before the first is consumed, instead of one round trip per element)
    // (state of a fresh latent: its sums are read all the same and replaced by zeros.  A load under "if the
    // latent is not fresh" waits for the latent's mu first: one trip to memory after the other, 8 + 16 of them here)
    float den0[CTA];
    {
        float mu_c[CTA], dn_c[CTA];
#pragma unroll
        for (int ct = 0; ct < CTA; ++ct) {
            mu_c[ct] = mu_g[ct * 16 + c16];
            dn_c[ct] = den_g[ct * 16 + c16];
        }
#pragma unroll
        for (int ct = 0; ct < CTA; ++ct) den0[ct] = mu_c[ct] <= kNegBig ? 0.f : dn_c[ct];
    }
    // state numerator of the wave's own latents: tile (mt, dt) holds rows m0 + 16 mt + 4g + r, column 16 dt + c16
    f32x4 U[MT][DT];
    {
        float mu_r[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) mu_r[mt][r] = mu_g[m0 + mt * 16 + 4 * g + r];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) U[mt][dt][r] = num_g[(int64_t)(m0 + mt * 16 + 4 * g + r) * D + dt * 16 + c16];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) U[mt][dt][r] = mu_r[mt][r] <= kNegBig ? 0.f : U[mt][dt][r];
    }
    for (int s = 0; s < n_before; ++s) {
        const float* sd = a.seg_den + ((int64_t)bh * a.n_slots + s) * M;
        const float* sn = a.seg_num + ((int64_t)bh * a.n_slots + s) * M * D;
        float td[CTA];
        f32x4 tu[MT][DT];
#pragma unroll
        for (int ct = 0; ct < CTA; ++ct) td[ct] = sd[ct * 16 + c16];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) tu[mt][dt][r] = sn[(int64_t)(m0 + mt * 16 + 4 * g + r) * D + dt * 16 + c16];
#pragma unroll
        for (int ct = 0; ct < CTA; ++ct) den0[ct] += td[ct];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) U[mt][dt] += tu[mt][dt];
    }

    uint2 ltri;
    {
        const uint32_t one = P_::kOnes2 & 0xffffu;
        uint32_t e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = (4 * g + i <= c16) ? one : 0u;
        ltri = make_uint2(e[0] | (e[1] << 16), e[2] | (e[3] << 16));
    }
    const f32x4 zf = {0.f, 0.f, 0.f, 0.f};

    static_assert(kChunk * (D / 8) == VPT * 256, "every thread stages the same number of V pieces");
    u32x4 ka[KD], kn[KD], vr[VPT];
    // K rows of the wave's 16 tokens and the thread's V pieces of a chunk; rows past the end of the segment repeat
    // its last row (their probabilities are zeroed where they are used).  No branch: see the main loop.
    auto load_chunk = [&](int n0, u32x4 (&kk)[KD]) {
        const int n = min(n0 + 16 * w + c16, N - 1);
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) kk[kd] = *reinterpret_cast<const u32x4*>(k + (int64_t)n * a.ks[2] + kd * 32 + g * 8);
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = tid + i * 256, tok = c / (D / 8), ch = c % (D / 8);
            vr[i] = *reinterpret_cast<const u32x4*>(v + (int64_t)min(n0 + tok, N - 1) * a.vs[2] + ch * 8);
        }
    };
    auto store_v = [&]() {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = tid + i * 256, tok = c / (D / 8), ch = c % (D / 8);
            u32x4 o = vr[i];
            if constexpr (!std::is_same<T, bf16_t>::value) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    o[j] = P_::pack2(M_::unpack(uint16_t(vr[i][j] & 0xffffu)), M_::unpack(uint16_t(vr[i][j] >> 16)));
            }
            *reinterpret_cast<u32x4*>(vs + tok * VS + ch * 8) = o;
        }
    };
    // the state of the wave's latents as B operands (k-slots = its 32 latents, lane = column d)
    auto publish_u = [&]() {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const f32x4 u0 = U[0][dt], u1 = U[1][dt];
            u0s[(w * DT + dt) * 64 + lane] = u32x4{P_::pack2(u0[0], u0[1]), P_::pack2(u0[2], u0[3]),
                                                   P_::pack2(u1[0], u1[1]), P_::pack2(u1[2], u1[3])};
        }
    };
    // Transposing reads: byte addresses in LDS of the lane's piece in a [latent][16 tokens] tile and in the V chunk; every
    // read adds a compile-time offset to one of these.
    const uint32_t lane_t = (4 * g + (c16 >> 2)) * 32 + (c16 & 3) * 8;
    const uint32_t pt_b = opaque((uint32_t)(uintptr_t)pt + lane_t);                  // P^T of wave 0
    const uint32_t ptw_b = opaque(pt_b + w * (M * 32)), gtw_b = opaque((uint32_t)(uintptr_t)gt + w * (M * 32) + lane_t);
    const uint32_t vs_b = opaque((uint32_t)(uintptr_t)vs + (4 * g + (c16 >> 2)) * (VS * 2) + (c16 & 3) * 8);    // V rows of wave 0's tokens
    const uint32_t vsw_b = opaque(vs_b + w * (16 * VS * 2));
    // ordinary reads: operand sets by lane, per-latent tables by column c16, P^T rows of the wave's own latents
    const uint32_t qs_b = opaque((uint32_t)(uintptr_t)qs + lane * 16), u0_b = opaque((uint32_t)(uintptr_t)u0s + lane * 16);
    const uint32_t cs_b = opaque((uint32_t)(uintptr_t)cs + c16 * 16), fo_b = opaque((uint32_t)(uintptr_t)fops + g * 16);
    const uint32_t mu_b = opaque((uint32_t)(uintptr_t)mu0s + c16 * 4);        // fws follows mu0s
    const uint32_t up_b = opaque((uint32_t)(uintptr_t)pt + (m0 + c16) * 32 + g * 8);
    // operands with tokens in lanes and latents in k-slots from a [latent][token] tile (k-step ks = 32 latents)
    auto tr_ops = [&](uint32_t tile_b, auto off_c, u32x4 (&o)[KS]) {
        constexpr int OFF = decltype(off_c)::value;
        static_assert(KS == 4, "four k-steps of 32 latents");
        const uint2 l0 = tr16_at<OFF>(tile_b), h0 = tr16_at<OFF + 512>(tile_b);
        const uint2 l1 = tr16_at<OFF + 1024>(tile_b), h1 = tr16_at<OFF + 1536>(tile_b);
        const uint2 l2 = tr16_at<OFF + 2048>(tile_b), h2 = tr16_at<OFF + 2560>(tile_b);
        const uint2 l3 = tr16_at<OFF + 3072>(tile_b), h3 = tr16_at<OFF + 3584>(tile_b);
        o[0] = u32x4{l0.x, l0.y, h0.x, h0.y};
        o[1] = u32x4{l1.x, l1.y, h1.x, h1.y};
        o[2] = u32x4{l2.x, l2.y, h2.x, h2.y};
        o[3] = u32x4{l3.x, l3.y, h3.x, h3.y};
    };
    // V rows of one wave's 16 tokens as B operands (token k-slots, lane = column d), DT column tiles
    auto v_ops = [&](uint32_t v_b, auto off_c, uint2 (&o)[DT]) {
        constexpr int OFF = decltype(off_c)::value;
        o[0] = tr16_at<OFF>(v_b);
        o[1] = tr16_at<OFF + 32>(v_b);
        if constexpr (DT == 4) {
            o[2] = tr16_at<OFF + 64>(v_b);
            o[3] = tr16_at<OFF + 96>(v_b);
        }
    };

    // Everything a step reads from LDS is requested in one batch ahead of the step and held in registers, with the
    // compiler kept from moving the requests next to their uses (it otherwise issues them one by one, each followed by a
    // wait: the chunk is a dependent chain, and with two waves per SIMD nothing else covers an LDS round trip).
    u32x4 qo[CTA][KD];      // q operands of the score product: constant, re-read per chunk (64 registers held all chunk long cost more)
    float mu0[CTA];
    auto load_q = [&]() {
        static_for<CTA>([&](auto ct_c) {
            constexpr int ct = decltype(ct_c)::value;
            mu0[ct] = lds_at<float, ct * 64>(mu_b);
            static_for<KD>([&](auto kd_c) {
                constexpr int kd = decltype(kd_c)::value;
                qo[ct][kd] = lds_at<u32x4, (ct * KD + kd) * 1024>(qs_b);
            });
        });
    };
    // operands of one 16-token tile of another wave against this wave's G: its P^T (A operands) and its V rows
    auto load_pair = [&](auto wp_c, u32x4 (&po)[KS], uint2 (&vo)[DT]) {
        constexpr int WP = decltype(wp_c)::value;
        tr_ops(pt_b, std::integral_constant<int, WP * M * 32>{}, po);
        v_ops(vs_b, std::integral_constant<int, WP * 16 * VS * 2>{}, vo);
    };

    bool bad = false;
    load_chunk(n_lo, ka);
    store_v();
    publish_u();
    __syncthreads();                                        // q operands

    for (int n0 = n_lo; n0 < N; n0 += kChunk) {
        load_q();
        const int tbase = n0 + 16 * w;
        const int tbw = min(16, max(0, N - tbase));        // valid tokens of this wave in the chunk
        // Tokens past the end of the segment (only its last chunk can have any) get probability 0 through the initial
        // value of their score accumulators: one quad per chunk, shared by the eight latent tiles.
        f32x4 absent;
#pragma unroll
        for (int r = 0; r < 4; ++r) absent[r] = (4 * g + r < tbw) ? 0.f : -1.0e30f;
        // The next chunk's K rows and V pieces are requested here, a whole chunk before they are handed over at the
        // bottom of the iteration (past the end of the segment the last rows are fetched again and never used).
        // Unconditional, so that the compiler's wait at the hand-over counts what is in flight instead of draining
        // whatever was issued last.
        load_chunk(n0 + kChunk, kn);

        // ---- token side, part 1: scores, P, column sums; publish P^T ----
        float p[CTA][4];
        uint2 ppk[CTA];
        f32x4 dc[CTA];
        {
            f32x4 sc[CTA];
#pragma unroll
            for (int ct = 0; ct < CTA; ++ct) {
                f32x4 s = absent;
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) s = M_::mma32(ka[kd], qo[ct][kd], s);
                sc[ct] = s;
            }
#pragma unroll
            for (int ct = 0; ct < CTA; ++ct) {
#pragma unroll
                for (int r = 0; r < 4; ++r) p[ct][r] = fast_exp2(sc[ct][r] - mu0[ct]);
                ppk[ct] = make_uint2(P_::pack2(p[ct][0], p[ct][1]), P_::pack2(p[ct][2], p[ct][3]));
            }
            // running sums over the wave's tokens (row t = 4g + r: tokens 0..t); the last row is the column sum
#pragma unroll
            for (int ct = 0; ct < CTA; ++ct) dc[ct] = P_::mma16(ltri, ppk[ct], zf);
#pragma unroll
            for (int ct = 0; ct < CTA; ++ct) {
                if (g == 3) cs[(ct * 16 + c16) * 4 + w] = dc[ct][3];
                *reinterpret_cast<uint2*>(ptw + (ct * 16 + c16) * 16 + 4 * g) = ppk[ct];
            }
        }
        __syncthreads();                                    // P^T, cs, V chunk, U0 operands visible

        // ---- token side, part 2: running denominators, G ----
        {
            f32x4 c4[CTA];
            float fw[CTA];      // the token's softmax weight over the latents is P * exp2(mu0 - cref)
            static_for<CTA>([&](auto ct_c) {
                constexpr int ct = decltype(ct_c)::value;
                c4[ct] = lds_at<f32x4, ct * 256>(cs_b);
                fw[ct] = lds_at<float, M * 4 + ct * 64>(mu_b);
            });
            FLARE_CHUNK_FENCE();
#pragma unroll
            for (int ct = 0; ct < CTA; ++ct) {
                float base = den0[ct];
                if (w > 0) base += c4[ct][0];
                if (w > 1) base += c4[ct][1];
                if (w > 2) base += c4[ct][2];
                den0[ct] = den0[ct] + c4[ct][0] + c4[ct][1] + c4[ct][2] + c4[ct][3];        // same order in every wave
                // dcum >= the element's own P; the smallest normal number added to it changes nothing unless dcum is 0
                // (or within 2^24 of that number), where it keeps the reciprocal finite and G = 0 where P = 0
                base += 1.17549435e-38f;
                float gv[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) gv[r] = p[ct][r] * fw[ct] * __builtin_amdgcn_rcpf(dc[ct][r] + base);
                *reinterpret_cast<uint2*>(gtw + (ct * 16 + c16) * 16 + 4 * g) = make_uint2(P_::pack2(gv[0], gv[1]), P_::pack2(gv[2], gv[3]));
            }
        }
        // operands of the outputs: G and P of the wave's tokens, the weight factors, U0 (two column tiles at a time), the
        // wave's own V rows, and the first of the earlier waves' tiles (w is uniform over the wave)
        u32x4 gop[KS], pop[KS], fo[KS], uo[2][KS];
        uint2 vd[DT];
        u32x4 pa[KS], pb[KS];
        uint2 va[DT], vb[DT];
        auto load_u0 = [&](auto half_c) {
            constexpr int h0 = decltype(half_c)::value * 2;
            static_for<KS>([&](auto ks_c) {
                constexpr int ks = decltype(ks_c)::value;
                uo[0][ks] = lds_at<u32x4, (ks * DT + h0) * 1024>(u0_b);
                uo[1][ks] = lds_at<u32x4, (ks * DT + h0 + 1) * 1024>(u0_b);
            });
        };
        tr_ops(gtw_b, std::integral_constant<int, 0>{}, gop);
        tr_ops(ptw_b, std::integral_constant<int, 0>{}, pop);
        static_for<KS>([&](auto ks_c) {
            constexpr int ks = decltype(ks_c)::value;
            fo[ks] = lds_at<u32x4, ks * 64>(fo_b);
        });
        load_u0(std::integral_constant<int, 0>{});
        FLARE_CHUNK_FENCE();
        // softmax sums over the latents of the wave's tokens (rows t = 4g + r, equal in every column)
        f32x4 rsum = zf;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) rsum = P_::mma32(pop[ks], fo[ks], rsum);

        // ---- outputs: G U0, then the chunk's own tokens up to and including this wave's ----
        f32x4 yacc[DT];
        auto g_u0 = [&](int d0) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                f32x4 acc = zf;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = P_::mma32(gop[ks], uo[j][ks], acc);
                yacc[d0 + j] = acc;
            }
        };
        g_u0(0);
        FLARE_CHUNK_FENCE();
        if constexpr (DT == 4) load_u0(std::integral_constant<int, 1>{});
        v_ops(vsw_b, std::integral_constant<int, 0>{}, vd);
        if (w > 0) load_pair(std::integral_constant<int, 0>{}, pa, va);
        FLARE_CHUNK_FENCE();
        if constexpr (DT == 4) g_u0(2);
        // [tau of wave wp, t of this wave] = sum_m P[tau,m] G[t,m], then times V of wave wp
        auto pair = [&](const u32x4 (&po)[KS], const uint2 (&vo)[DT], bool diag) {
            f32x4 acct = zf;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) acct = P_::mma32(po[ks], gop[ks], acct);
            if (diag) {
#pragma unroll
                for (int r = 0; r < 4; ++r) acct[r] = (4 * g + r <= c16) ? acct[r] : 0.f;
            }
            const uint2 aop = make_uint2(P_::pack2(acct[0], acct[1]), P_::pack2(acct[2], acct[3]));
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) yacc[dt] = P_::mma16(aop, vo[dt], yacc[dt]);
        };
        {
            if (w > 1) load_pair(std::integral_constant<int, 1>{}, pb, vb);
            FLARE_CHUNK_FENCE();
            if (w > 0) {
                pair(pa, va, false);
                if (w > 2) load_pair(std::integral_constant<int, 2>{}, pa, va);
                FLARE_CHUNK_FENCE();
                if (w > 1) {
                    pair(pb, vb, false);
                    if (w > 2) pair(pa, va, false);
                }
            }
            pair(pop, vd, true);
        }
        // operands of the state update (P^T of all four waves at this wave's latents, V of the whole chunk): requested ahead
        // of the output's trip through LDS
        uint2 uv[4][DT], up[4][MT];
        v_ops(vs_b, std::integral_constant<int, 0>{}, uv[0]);
        v_ops(vs_b, std::integral_constant<int, 16 * VS * 2>{}, uv[1]);
        v_ops(vs_b, std::integral_constant<int, 32 * VS * 2>{}, uv[2]);
        v_ops(vs_b, std::integral_constant<int, 48 * VS * 2>{}, uv[3]);
        static_for<4>([&](auto wp_c) {
            constexpr int wp = decltype(wp_c)::value;
            static_for<MT>([&](auto mt_c) {
                constexpr int mt = decltype(mt_c)::value;
                const u32v2 t = lds_at<u32v2, wp * M * 32 + mt * 512>(up_b);
                up[wp][mt] = make_uint2(t[0], t[1]);
            });
        });
        FLARE_CHUNK_FENCE();
        // The next chunk's rows, requested at the top of this iteration, are waited for here, before the stores below
        // are issued: loads and stores complete in order on one counter, the stores sit under per-lane conditions, and
        // a wait placed at the hand-over after them could only wait for everything, store acknowledgements included.
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        // y rows / softmax sums, transposed through the wave's (now free) G^T region: lane (g, c16) ends
        // up with y[token c16][16 dt + 4g .. 4g + 3]
        {
            float inv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                inv[r] = __builtin_amdgcn_rcpf(rsum[r]);
                if (4 * g + r < tbw) {
                    bad = bad || !(rsum[r] >= kLMin && rsum[r] <= kLMax);
                    if (a.lse && c16 == 0) a.lse[(int64_t)bh * a.N + tbase + 4 * g + r] = (cref + __log2f(rsum[r])) * kLn2;
                }
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    o[r] = yacc[dt][r] * inv[r];
                    if (4 * g + r < tbw) bad = bad || !(fabsf(o[r]) <= 3.0e38f);
                }
                *reinterpret_cast<uint2*>(gtw + (dt * 16 + c16) * 16 + 4 * g) = make_uint2(M_::pack2(o[0], o[1]), M_::pack2(o[2], o[3]));
            }
        }
        uint2 yo[DT];
        yo[0] = tr16_at<0>(gtw_b);
        yo[1] = tr16_at<512>(gtw_b);
        if constexpr (DT == 4) {
            yo[2] = tr16_at<1024>(gtw_b);
            yo[3] = tr16_at<1536>(gtw_b);
        }
        FLARE_CHUNK_FENCE();

        // ---- state update of the wave's own latents over all 64 tokens (covers the transposition's round trip) ----
        // Two waves' tokens share one product over 32 tokens: k-slot 8g + j of the 16x16x32 instruction holds token 4g + j of
        // the first wave for j < 4 and token 4g + j - 4 of the second otherwise, on both operands.
#pragma unroll
        for (int h2 = 0; h2 < 4; h2 += 2)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const u32x4 pa2 = u32x4{up[h2][mt].x, up[h2][mt].y, up[h2 + 1][mt].x, up[h2 + 1][mt].y};
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    U[mt][dt] = P_::mma32(pa2, u32x4{uv[h2][dt].x, uv[h2][dt].y, uv[h2 + 1][dt].x, uv[h2 + 1][dt].y}, U[mt][dt]);
            }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            if (c16 < tbw) *reinterpret_cast<uint2*>(y + (int64_t)(tbase + c16) * a.ys[2] + dt * 16 + 4 * g) = yo[dt];

        __syncthreads();                                    // everyone is done with V, U0, P^T of this chunk
        if (n0 + kChunk < N) {
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) ka[kd] = kn[kd];
            store_v();
            publish_u();
        }
    }

    const bool last = seg == a.n_segs - 1;
#pragma unroll
    for (int ct = 0; ct < CTA; ++ct) bad = bad || (last && !(den0[ct] >= kLMin && den0[ct] <= kLMax));
    if (__any(bad) && lane == 0) bad_flag = 1;
    __syncthreads();
    if (bad_flag) {
        if (tid == 0) a.flags[bh] = 1;
        return;
    }
    if (single && tid == 0) a.flags[bh] = 0;
    if (!last) return;
    float* den_o = single ? den_g : seg_den;
    float* num_o = single ? num_g : seg_num;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int ct = 2 * w + mt, m = ct * 16 + c16;
        if (g == 0) {
            if (single) mu_g[m] = mu0s[m] * kLn2;
            den_o[m] = den0[ct];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) num_o[(int64_t)(m0 + mt * 16 + 4 * g + r) * D + dt * 16 + c16] = U[mt][dt][r];
    }
}

template <typename T, bool STATE_ONLY>
hipError_t launch_phase(const CausalArgs& a, int step, dim3 grid, hipStream_t st)
{
    dim3 block(256);
    if (a.D == 64 && a.M == 128)      hipLaunchKernelGGL((causal_mfma_kernel<T, 64, 1, STATE_ONLY>), grid, block, 0, st, a, step);
    else if (a.D == 32 && a.M == 128) hipLaunchKernelGGL((causal_mfma_kernel<T, 32, 1, STATE_ONLY>), grid, block, 0, st, a, step);
    else if (a.D == 32 && a.M == 256) hipLaunchKernelGGL((causal_mfma_kernel<T, 32, 2, STATE_ONLY>), grid, block, 0, st, a, step);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_chunk_d(const CausalArgs& a, dim3 grid, hipStream_t st)
{
    auto kern = causal_chunk_kernel<T, D>;
    constexpr size_t lds = causal_chunk_lds<D>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a);
    return hipGetLastError();
}

// The recurrence phase: 64-token chunks for the prefill at M = 128, 16-token (or 1-token) blocks otherwise.
template <typename T>
hipError_t launch_recurrence(const CausalArgs& a, int step, dim3 grid, hipStream_t st)
{
    if (step == kTB && a.M == 128) return a.D == 64 ? launch_chunk_d<T, 64>(a, grid, st) : launch_chunk_d<T, 32>(a, grid, st);
    return launch_phase<T, false>(a, step, grid, st);
}

template <typename T>
hipError_t launch_t(const CausalArgs& a, int step, hipStream_t st)
{
    const int BH = a.B * a.H;
    if (a.n_segs == 1) return launch_recurrence<T>(a, step, dim3(BH, 1), st);
    // the first phase also clears the redo flags and segment counters
    hipError_t e = launch_phase<T, true>(a, step, dim3(BH, a.n_pieces), st);
    if (e != hipSuccess) return e;
    // The last segment has staged the final state in the workspace; the fp32 kernel launched behind this one copies
    // it into (mu, den, num) for every (b,h) whose flag stayed clear and redoes the others from their incoming state.
    return launch_recurrence<T>(a, step, dim3(BH, a.n_segs), st);
}

}  // namespace

bool causal_mfma_supported(int dtype, int M, int D)
{
    // the fp32 kernel must be able to redo any (b,h), so its LDS limit applies here too
    return (dtype == 1 || dtype == 2) && (D == 32 || D == 64) && (M == 128 || M == 256) &&
           causal_lds_bytes(M, D, false) <= 160 * 1024;
}

hipError_t launch_causal_mfma(const CausalArgs& a, int dtype, int step, hipStream_t st)
{
    if (step == 1) return launch_causal_decode_steps(a, dtype, st);      // a decode step has no matrix shape
    return dtype == 1 ? launch_t<bf16_t>(a, step, st) : launch_t<f16_t>(a, step, st);
}

}  // namespace flare
