// Triple (third-order) linear attention on the matrix cores: bf16 / f16, head dims that are multiples of 16 up to 64
// (both contractions are sums over blocks of 16 indices; the text below describes one 16 x 16 x 16 block).
//
//   state[i,j,k] = (1/N) sum_n f(k1)[n,i] v[n,j] f(k2)[n,k]      (lra/models/backends.py:1289 of the reference)
//   out[n,j]     = sum_{i,k} f(q1)[n,i] state[i,j,k] f(q2)[n,k]  (backends.py:1290)
// For a fixed k both contractions are 16x16x16 products:
//   state[:, :, k] += A_k^T V     with A_k[n,i] = f(k1)[n,i] f(k2)[n,k]           (contraction over 16 tokens)
//   T_k[n,:]        = f(q1)[n,:] state[:, :, k] ;  out[n,:] += T_k[n,:] f(q2)[n,k] (contraction over i)
// so a wave walks 16-token tiles with v_mfma_f32_16x16x16.  The state kernel stages its tiles (feature map
// applied, rounded to the element type) in a wave-private LDS tile and takes them with tokens in the k-slots
// through the LDS transpose read; the output kernel reads f(q1) straight from global memory as a B operand.
// No barrier in the token loops and no atomics: a workgroup sums its four waves in a fixed order and writes one
// split partial; the fixed-order merge of triple.hip sums the partials.
#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Tm;
template <> struct Tm<bf16_t> {
    static __device__ __forceinline__ f32x4 mma16(uint2 a, uint2 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
};
template <> struct Tm<f16_t> {
    static __device__ __forceinline__ f32x4 mma16(uint2 a, uint2 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float lo(uint32_t w) { return float(__builtin_bit_cast(f16x2, w)[0]); }
    static __device__ __forceinline__ float hi(uint32_t w) { return float(__builtin_bit_cast(f16x2, w)[1]); }
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

__device__ __forceinline__ float featf(float x, int fm)
{
    if (!fm) return x;
    return x > 0.f ? x + 1.f : __expf(x);
}

// 4 elements (8 bytes, already in registers) -> feature map -> repacked; `live` = false gives zeros
template <typename T>
__device__ __forceinline__ uint2 feat4_of(uint2 raw, bool live, int fm)
{
    uint2 f = raw;
    if (fm)
        f = make_uint2(Tm<T>::pack2(featf(Tm<T>::lo(raw.x), fm), featf(Tm<T>::hi(raw.x), fm)),
                       Tm<T>::pack2(featf(Tm<T>::lo(raw.y), fm), featf(Tm<T>::hi(raw.y), fm)));
    return make_uint2(live ? f.x : 0u, live ? f.y : 0u);
}

// Sum over the 16 lanes of a row with DPP operands (vector ALU only): pairs, quads, half rows, the row.
template <int CTRL> __device__ __forceinline__ float dpp_of(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_sum(float x)
{
    x += dpp_of<0xB1>(x);      // quad_perm [1,0,3,2]
    x += dpp_of<0x4E>(x);      // quad_perm [2,3,0,1]
    x += dpp_of<0x141>(x);     // row_half_mirror
    x += dpp_of<0x140>(x);     // row_mirror
    return x;
}

constexpr int kD = 16;

// x * (the value y has in lane (c - R) mod 16 of the same 16-lane row): one vector instruction with a DPP row
// rotate on its first operand.  The DPP read of a freshly written register needs two wait states that the compiler
// does not insert for assembly it cannot see into: the caller provides them (see the state kernel's tile).
template <int R> __device__ __forceinline__ float mul_row_ror(float x, float y)
{
    if constexpr (R == 0) {
        return x * y;
    } else {
        float d;
        asm("v_mul_f32_dpp %0, %1, %2 row_ror:%3 row_mask:0xf bank_mask:0xf" : "=v"(d) : "v"(y), "v"(x), "i"(R));
        return d;
    }
}

constexpr size_t kStateRedBytes = 4 * (kD + 1) * 64 * 4 * sizeof(float);

// grid (n_splits * blocks, H, B), blocks = (Dq/16)^2 (Dv/16) blocks of 16 x 16 x 16 state entries (one for head dims
// of 16); wave w of a workgroup takes the 16-token tiles w, w+4, ... of the split.
//
// Per tile the wave stages f(k1), f(k2), v (rounded to the element type) in its own LDS tile and takes all three
// with tokens in the k-slots (transpose read: lane = feature c16, slots = tokens 4g..4g+3).  The state is
// accumulated along "diagonals": step r multiplies the lane's f(k1)[n, i = c16] by f(k2)[n, (c16 - r) mod 16],
// which is the value its neighbour r lanes down the row holds (a DPP rotate inside the multiply: no LDS read,
// no broadcast), so S[r][i][j] = state[i][j][(i - r) mod 16].  The four waves meet once, at the end.
template <typename T>
__global__ __launch_bounds__(256, 2) void triple_state_mfma_kernel(TripleArgs a)
{
    using M_ = Tm<T>;
    __shared__ __attribute__((aligned(16))) uint16_t k1s[4][16][kD];
    __shared__ __attribute__((aligned(16))) uint16_t k2s[4][16][kD];
    __shared__ __attribute__((aligned(16))) uint16_t vs[4][16][kD];
    extern __shared__ __attribute__((aligned(16))) uint8_t triple_red[];      // kStateRedBytes: where the waves meet
    float (*red)[kD + 1][64][4] = reinterpret_cast<float (*)[kD + 1][64][4]>(triple_red);

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    // the workgroup's 16 x 16 x 16 block of the state: rows i of block ib, columns j of block jb, slices k of block kb
    const int nbq = a.Dq >> 4, nbv = a.Dv >> 4, NB = nbq * nbv * nbq;
    const int split = blockIdx.x / NB, blk = blockIdx.x % NB, h = blockIdx.y, b = blockIdx.z;
    const int ib = blk / (nbv * nbq), jb = (blk / nbq) % nbv, kb = blk % nbq;
    const uint16_t* k1 = (const uint16_t*)a.k1 + b * a.k1s[0] + h * a.k1s[1] + 16 * ib;
    const uint16_t* k2 = (const uint16_t*)a.k2 + b * a.k2s[0] + h * a.k2s[1] + 16 * kb;
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1] + 16 * jb;
    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int tok = lane >> 2, piece = (lane & 3) * 4;   // staging: lane = (token, 4 elements)

    f32x4 S[kD], kk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < kD; ++k) S[k] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Raw 8-byte pieces of the tiles two ahead are fetched while the current one is processed.  The loads are
    // unconditional (rows past the end repeat the last row and are zeroed when staged): with no branch around a
    // memory instruction the compiler's waits count exactly what is in flight instead of draining everything.
    auto fetch = [&](int n0, uint2& r1, uint2& r2, uint2& rv) {
        const int n = min(n0 + tok, n_end - 1);
        r1 = *reinterpret_cast<const uint2*>(k1 + (int64_t)n * a.k1s[2] + piece);
        r2 = *reinterpret_cast<const uint2*>(k2 + (int64_t)n * a.k2s[2] + piece);
        rv = *reinterpret_cast<const uint2*>(v + (int64_t)n * a.vs[2] + piece);
    };
    auto feat4 = [&](uint2 raw, bool live) {
        uint2 f = raw;
        if (a.feature_map)
            f = make_uint2(M_::pack2(featf(M_::lo(raw.x), 1), featf(M_::hi(raw.x), 1)),
                           M_::pack2(featf(M_::lo(raw.y), 1), featf(M_::hi(raw.y), 1)));
        return make_uint2(live ? f.x : 0u, live ? f.y : 0u);
    };
    auto step = [&](auto r_c, const float (&k1f)[4], const float (&k2f)[4], uint2 vt) {
        constexpr int R = decltype(r_c)::value;
        const uint2 ak = make_uint2(M_::pack2(mul_row_ror<R>(k1f[0], k2f[0]), mul_row_ror<R>(k1f[1], k2f[1])),
                                    M_::pack2(mul_row_ror<R>(k1f[2], k2f[2]), mul_row_ror<R>(k1f[3], k2f[3])));
        S[R] = M_::mma16(ak, vt, S[R]);
    };
    // one tile: stage (c1, c2, cv), then the seventeen products
    auto tile = [&](int n0, uint2 c1, uint2 c2, uint2 cv) {
        const bool live = n0 + tok < n_end;
        *reinterpret_cast<uint2*>(&k1s[w][tok][piece]) = feat4(c1, live);
        *reinterpret_cast<uint2*>(&k2s[w][tok][piece]) = feat4(c2, live);
        *reinterpret_cast<uint2*>(&vs[w][tok][piece]) = make_uint2(live ? cv.x : 0u, live ? cv.y : 0u);
        // tokens 4g..4g+3 in the k-slots, lane = feature index c16
        const int tr_row = 4 * g + (c16 >> 2), tr_col = (c16 & 3) * 4;
        const uint2 k1t = tr16(&k1s[w][tr_row][tr_col]);
        const uint2 k2t = tr16(&k2s[w][tr_row][tr_col]);
        const uint2 vt = tr16(&vs[w][tr_row][tr_col]);
        kk = M_::mma16(k1t, k2t, kk);
        const float k1f[4] = {M_::lo(k1t.x), M_::hi(k1t.x), M_::lo(k1t.y), M_::hi(k1t.y)};
        float k2f[4] = {M_::lo(k2t.x), M_::hi(k2t.x), M_::lo(k2t.y), M_::hi(k2t.y)};
        // The DPP reads of k2f below sit in assembly the compiler does not look into, so it cannot place the two wait
        // states a DPP read needs after the instruction that wrote the register: this statement "rewrites" the four
        // factors (nothing may move across it) and spends those wait states once per tile.
        asm volatile("s_nop 1" : "+v"(k2f[0]), "+v"(k2f[1]), "+v"(k2f[2]), "+v"(k2f[3]));
        step(std::integral_constant<int, 0>{}, k1f, k2f, vt);   step(std::integral_constant<int, 1>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 2>{}, k1f, k2f, vt);   step(std::integral_constant<int, 3>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 4>{}, k1f, k2f, vt);   step(std::integral_constant<int, 5>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 6>{}, k1f, k2f, vt);   step(std::integral_constant<int, 7>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 8>{}, k1f, k2f, vt);   step(std::integral_constant<int, 9>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 10>{}, k1f, k2f, vt);  step(std::integral_constant<int, 11>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 12>{}, k1f, k2f, vt);  step(std::integral_constant<int, 13>{}, k1f, k2f, vt);
        step(std::integral_constant<int, 14>{}, k1f, k2f, vt);  step(std::integral_constant<int, 15>{}, k1f, k2f, vt);
    };
    // three register sets take turns: a set is refilled with the tile three ahead as soon as its tile is staged,
    // so no register is copied from one set to another (a copy would have to wait for the load it copies)
    uint2 a1, a2, av, b1, b2, bv, c1, c2, cv;
    int n0 = n_begin + w * 16;
    if (n0 < n_end) {
        fetch(n0, a1, a2, av);
        fetch(n0 + 64, b1, b2, bv);
        fetch(n0 + 128, c1, c2, cv);
        for (;; n0 += 192) {
            { const uint2 t1 = a1, t2 = a2, tv = av; fetch(n0 + 192, a1, a2, av); tile(n0, t1, t2, tv); }
            if (n0 + 64 >= n_end) break;
            { const uint2 t1 = b1, t2 = b2, tv = bv; fetch(n0 + 256, b1, b2, bv); tile(n0 + 64, t1, t2, tv); }
            if (n0 + 128 >= n_end) break;
            { const uint2 t1 = c1, t2 = c2, tv = cv; fetch(n0 + 320, c1, c2, cv); tile(n0 + 128, t1, t2, tv); }
            if (n0 + 192 >= n_end) break;
        }
    }

    // the four waves' accumulators meet in LDS once; wave w then sums steps 4w..4w+3 (and wave 0 the normaliser
    // state) over the waves in a fixed order and writes its share of the workgroup's partial
#pragma unroll
    for (int k = 0; k < kD; ++k) *reinterpret_cast<f32x4*>(&red[w][k][lane][0]) = S[k];
    *reinterpret_cast<f32x4*>(&red[w][kD][lane][0]) = kk;
    __syncthreads();
    const size_t per = (size_t)kD * kD * kD + (size_t)kD * kD;
    float* part = a.part + ((((size_t)b * a.H + h) * a.n_parts + split) * NB + blk) * per;
    // The partial keeps the accumulators' own order, [step r][lane][register rr] (and the normaliser tile behind
    // them), so that every store is 16 contiguous bytes per lane; the merge kernel puts the sums into [i][j][k].
#pragma unroll
    for (int rr4 = 0; rr4 < 4; ++rr4) {
        const int r = 4 * w + rr4;
        const f32x4 t = *reinterpret_cast<const f32x4*>(&red[0][r][lane][0]) + *reinterpret_cast<const f32x4*>(&red[1][r][lane][0]) +
                        *reinterpret_cast<const f32x4*>(&red[2][r][lane][0]) + *reinterpret_cast<const f32x4*>(&red[3][r][lane][0]);
        *reinterpret_cast<f32x4*>(part + ((size_t)r * 64 + lane) * 4) = t;
    }
    if (w == 0) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(&red[0][kD][lane][0]) + *reinterpret_cast<const f32x4*>(&red[1][kD][lane][0]) +
                        *reinterpret_cast<const f32x4*>(&red[2][kD][lane][0]) + *reinterpret_cast<const f32x4*>(&red[3][kD][lane][0]);
        *reinterpret_cast<f32x4*>(part + ((size_t)kD * 64 + lane) * 4) = t;
    }
}

// grid (ceil(N / tokens_per_wg), H, B); each wave walks 16-token tiles of the workgroup's range.
//
// The products are taken transposed, T_k^T[j, n] = sum_i state[i,j,k] f(q1)[n,i]: the state slices are the A
// operands (row j = c16, slots i = 4g..4g+3, set up once), f(q1) rows are the B operands straight from global
// memory (lane = token c16, slots i = 4g..4g+3: 8 contiguous bytes of the token's row), and the result has the
// token in the lane, so the factor f(q2)[n,k] is a per-lane scalar.  Only f(q2) passes through (wave-private) LDS,
// to hand every lane its token's sixteen features.
template <typename T>
__global__ __launch_bounds__(256) void triple_out_mfma_kernel(TripleArgs a, int tokens_per_wg)
{
    using M_ = Tm<T>;
    constexpr int QS = kD + 4;                                          // row stride of the f(q2) tile in floats
    __shared__ __attribute__((aligned(16))) float q2f[4][16][QS];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const uint16_t* q1 = (const uint16_t*)a.q1 + b * a.q1s[0] + h * a.q1s[1];
    const uint16_t* q2 = (const uint16_t*)a.q2 + b * a.q2s[0] + h * a.q2s[1];
    uint16_t* out = (uint16_t*)a.out + b * a.os[0] + h * a.os[1];
    const float* state = a.state + bh * kD * kD * kD;
    const int tok = lane >> 2, piece = (lane & 3) * 4;

    // A operands: sk[k] = state[i = 4g..4g+3][j = c16][k], kkb = kk[i = 4g..4g+3][k' = c16]
    uint2 sk[kD], kkb = make_uint2(0u, 0u);
    {
        float sv[4][kD];
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int k4 = 0; k4 < kD; k4 += 4) {
                const f32x4 t = *reinterpret_cast<const f32x4*>(state + ((size_t)(4 * g + e) * kD + c16) * kD + k4);
                sv[e][k4] = t[0]; sv[e][k4 + 1] = t[1]; sv[e][k4 + 2] = t[2]; sv[e][k4 + 3] = t[3];
            }
#pragma unroll
        for (int k = 0; k < kD; ++k) sk[k] = make_uint2(M_::pack2(sv[0][k], sv[1][k]), M_::pack2(sv[2][k], sv[3][k]));
        if (a.normalize) {
            const float* kkp = a.kk + bh * kD * kD;
            kkb = make_uint2(M_::pack2(kkp[(4 * g + 0) * kD + c16], kkp[(4 * g + 1) * kD + c16]),
                             M_::pack2(kkp[(4 * g + 2) * kD + c16], kkp[(4 * g + 3) * kD + c16]));
        }
    }

    const int wg_n0 = blockIdx.x * tokens_per_wg;
    const int wg_n1 = min(a.N, wg_n0 + tokens_per_wg);
    // Raw pieces of the tiles two ahead are fetched while the current one is being worked on: q1 as this lane's B
    // operand (token c16, features 4g..4g+3), q2 as the lane's share of the tile (token tok, features piece..).
    // Unconditional loads (rows past the end repeat the last row): no branch around a memory instruction, so the
    // compiler's waits count what is in flight.
    auto fetch = [&](int n0, uint2& r1, uint2& r2) {
        r1 = *reinterpret_cast<const uint2*>(q1 + (int64_t)min(n0 + c16, wg_n1 - 1) * a.q1s[2] + 4 * g);
        r2 = *reinterpret_cast<const uint2*>(q2 + (int64_t)min(n0 + tok, wg_n1 - 1) * a.q2s[2] + piece);
    };
    auto tile = [&](int n0, uint2 r1, uint2 r2) {
        const uint2 f2 = feat4_of<T>(r2, n0 + tok < wg_n1, a.feature_map);
        // (to the compiler every lane is a thread of its own: without the two fences it may move a lane's reads of other
        // lanes' rows across that lane's own store)
        asm volatile("" ::: "memory");
        *reinterpret_cast<f32x4*>(&q2f[w][tok][piece]) = f32x4{M_::lo(f2.x), M_::hi(f2.x), M_::lo(f2.y), M_::hi(f2.y)};
        asm volatile("" ::: "memory");
        const uint2 q1b = feat4_of<T>(r1, n0 + c16 < wg_n1, a.feature_map);
        // the sixteen f(q2) of the lane's token (the tile is private to the wave: reads follow its writes in program order)
        float r[kD];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(&q2f[w][c16][4 * c]);
            r[4 * c] = t[0]; r[4 * c + 1] = t[1]; r[4 * c + 2] = t[2]; r[4 * c + 3] = t[3];
        }
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};   // out[n = c16][j = 4g + e]
#pragma unroll
        for (int k = 0; k < kD; ++k) {
            const f32x4 t = M_::mma16(sk[k], q1b, f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = fmaf(t[e], r[k], acc[e]);
        }
        if (a.normalize) {
            // den[n] = sum_k' (sum_i kk[i,k'] f(q1)[n,i]) f(q2)[n,k']: the lane holds k' = 4g..4g+3 of its token
            const f32x4 wv = M_::mma16(kkb, q1b, f32x4{0.f, 0.f, 0.f, 0.f});
            const f32x4 rq = *reinterpret_cast<const f32x4*>(&q2f[w][c16][4 * g]);
            float den = wv[0] * rq[0] + wv[1] * rq[1] + wv[2] * rq[2] + wv[3] * rq[3];
            den = sum_xor32(sum_xor16(den));
            const float inv = 1.f / den;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] *= inv;
        }
        if (n0 + c16 < wg_n1)
            *reinterpret_cast<uint2*>(out + (int64_t)(n0 + c16) * a.os[2] + 4 * g) =
                make_uint2(M_::pack2(acc[0], acc[1]), M_::pack2(acc[2], acc[3]));
    };
    // three register sets take turns, each refilled with the tile three ahead once its own has been taken
    uint2 a1, a2, b1, b2, c1, c2;
    int n0 = wg_n0 + w * 16;
    if (n0 < wg_n1) {
        fetch(n0, a1, a2);
        fetch(n0 + 64, b1, b2);
        fetch(n0 + 128, c1, c2);
        for (;; n0 += 192) {
            { const uint2 t1 = a1, t2 = a2; fetch(n0 + 192, a1, a2); tile(n0, t1, t2); }
            if (n0 + 64 >= wg_n1) break;
            { const uint2 t1 = b1, t2 = b2; fetch(n0 + 256, b1, b2); tile(n0 + 64, t1, t2); }
            if (n0 + 128 >= wg_n1) break;
            { const uint2 t1 = c1, t2 = c2; fetch(n0 + 320, c1, c2); tile(n0 + 128, t1, t2); }
            if (n0 + 192 >= wg_n1) break;
        }
    }
}

// Head dims that are larger multiples of 16 (up to 64).  grid (ceil(N / tokens_per_wg) * Dv/16, H, B): a workgroup
// produces 16 output columns (block jb) for its token range.  The contraction over (i, k) runs over (Dq/16)^2 pairs
// of index blocks; their state slices sit in LDS as A operands (built once per workgroup), f(q1) pieces come
// straight from global memory as B operands, and f(q2) of the wave's tile passes through a wave-private LDS tile
// that hands every lane its token's features.
template <typename T>
__global__ __launch_bounds__(256) void triple_out_blocks_kernel(TripleArgs a, int tokens_per_wg)
{
    using M_ = Tm<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t triple_out_lds[];
    const int Dq = a.Dq, Dv = a.Dv, nbq = Dq >> 4, nbv = Dv >> 4, NP = nbq * nbq, QS = Dq + 4;
    uint2* skt = reinterpret_cast<uint2*>(triple_out_lds);                 // [pair][k][lane]
    uint2* kkt = skt + (size_t)NP * kD * 64;                                // [pair][lane]
    float* q2f = reinterpret_cast<float*>(kkt + (size_t)NP * 64);           // [wave][16][QS]

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int jb = blockIdx.x % nbv, wgx = blockIdx.x / nbv, h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const uint16_t* q1 = (const uint16_t*)a.q1 + b * a.q1s[0] + h * a.q1s[1];
    const uint16_t* q2 = (const uint16_t*)a.q2 + b * a.q2s[0] + h * a.q2s[1];
    uint16_t* out = (uint16_t*)a.out + b * a.os[0] + h * a.os[1] + 16 * jb;
    const float* state = a.state + bh * Dq * Dv * Dq;
    const float* kkp = a.kk + bh * Dq * Dq;
    float* q2w = q2f + (size_t)w * 16 * QS;

    // operand tables: entry (pair = ib nbq + kb, k, lane) = state[16 ib + 4g + e][16 jb + c16][16 kb + k], e = 0..3
    for (int idx = tid; idx < NP * kD * 64; idx += 256) {
        const int ln = idx & 63, k = (idx >> 6) & 15, pair = idx >> 10;
        const int ibb = pair / nbq, kbb = pair % nbq, gg = ln >> 4, cc = ln & 15;
        const float* s0 = state + ((size_t)(16 * ibb + 4 * gg) * Dv + 16 * jb + cc) * Dq + 16 * kbb + k;
        const size_t rs = (size_t)Dv * Dq;
        skt[idx] = make_uint2(M_::pack2(s0[0], s0[rs]), M_::pack2(s0[2 * rs], s0[3 * rs]));
    }
    if (a.normalize)
        for (int idx = tid; idx < NP * 64; idx += 256) {
            const int ln = idx & 63, pair = idx >> 6;
            const int ibb = pair / nbq, kbb = pair % nbq, gg = ln >> 4, cc = ln & 15;
            const float* s0 = kkp + (size_t)(16 * ibb + 4 * gg) * Dq + 16 * kbb + cc;
            kkt[idx] = make_uint2(M_::pack2(s0[0], s0[Dq]), M_::pack2(s0[2 * Dq], s0[3 * Dq]));
        }
    __syncthreads();

    const int wg_n0 = wgx * tokens_per_wg;
    const int wg_n1 = min(a.N, wg_n0 + tokens_per_wg);
    const int tok = lane >> 2, piece = (lane & 3) * 4;
    for (int n0 = wg_n0 + w * 16; n0 < wg_n1; n0 += 64) {
        // raw pieces of the tile: q1 as B operands (token c16, features 16 ib + 4g..), q2 as the lane's share of the tile
        uint2 r1[4], r2[4];
        const uint16_t* q1r = q1 + (int64_t)min(n0 + c16, wg_n1 - 1) * a.q1s[2] + 4 * g;
        const uint16_t* q2r = q2 + (int64_t)min(n0 + tok, wg_n1 - 1) * a.q2s[2] + piece;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < nbq) {
                r1[i] = *reinterpret_cast<const uint2*>(q1r + 16 * i);
                r2[i] = *reinterpret_cast<const uint2*>(q2r + 16 * i);
            }
        asm volatile("" ::: "memory");      // the lanes' stores and their reads of each other's rows keep their order
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < nbq) {
                const uint2 f2 = feat4_of<T>(r2[i], n0 + tok < wg_n1, a.feature_map);
                *reinterpret_cast<f32x4*>(q2w + tok * QS + 16 * i + piece) = f32x4{M_::lo(f2.x), M_::hi(f2.x), M_::lo(f2.y), M_::hi(f2.y)};
            }
        asm volatile("" ::: "memory");
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};   // out[n = c16][j = 16 jb + 4g + e]
        float den = 0.f;
        for (int ibb = 0; ibb < nbq; ++ibb) {
            uint2 raw = r1[0];
#pragma unroll
            for (int i = 1; i < 4; ++i) raw = ibb == i ? r1[i] : raw;
            const uint2 q1b = feat4_of<T>(raw, n0 + c16 < wg_n1, a.feature_map);
            for (int kbb = 0; kbb < nbq; ++kbb) {
                const int pair = ibb * nbq + kbb;
                float r[kD];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const f32x4 t = *reinterpret_cast<const f32x4*>(q2w + c16 * QS + 16 * kbb + 4 * c);
                    r[4 * c] = t[0]; r[4 * c + 1] = t[1]; r[4 * c + 2] = t[2]; r[4 * c + 3] = t[3];
                }
                const uint2* sk = skt + (size_t)pair * kD * 64 + lane;
#pragma unroll
                for (int k = 0; k < kD; ++k) {
                    const f32x4 t = M_::mma16(sk[k * 64], q1b, f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] = fmaf(t[e], r[k], acc[e]);
                }
                if (a.normalize) {
                    const f32x4 wv = M_::mma16(kkt[pair * 64 + lane], q1b, f32x4{0.f, 0.f, 0.f, 0.f});
                    const f32x4 rq = *reinterpret_cast<const f32x4*>(q2w + c16 * QS + 16 * kbb + 4 * g);
                    den += wv[0] * rq[0] + wv[1] * rq[1] + wv[2] * rq[2] + wv[3] * rq[3];
                }
            }
        }
        if (a.normalize) {
            const float inv = 1.f / sum_xor32(sum_xor16(den));
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] *= inv;
        }
        if (n0 + c16 < wg_n1)
            *reinterpret_cast<uint2*>(out + (int64_t)(n0 + c16) * a.os[2] + 4 * g) =
                make_uint2(M_::pack2(acc[0], acc[1]), M_::pack2(acc[2], acc[3]));
    }
}

}  // namespace

// 16-bit inputs, both head dims multiples of 16 up to 64
bool triple_mfma_supported(int dtype, int Dq, int Dv)
{
    return (dtype == 1 || dtype == 2) && Dq % 16 == 0 && Dv % 16 == 0 && Dq >= 16 && Dv >= 16 && Dq <= 64 && Dv <= 64;
}

hipError_t launch_triple_state_mfma(const TripleArgs& a, int dtype, hipStream_t st)
{
    dim3 grid(a.n_splits * (a.Dq / 16) * (a.Dv / 16) * (a.Dq / 16), a.H, a.B);
    auto kern = dtype == 1 ? triple_state_mfma_kernel<bf16_t> : triple_state_mfma_kernel<f16_t>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kStateRedBytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(256), kStateRedBytes, st, a);
    return hipGetLastError();
}

hipError_t launch_triple_out_mfma(const TripleArgs& a, int dtype, hipStream_t st)
{
    // ~8 workgroups per CU over the grid, ranges a multiple of 64 tokens
    const int64_t per_bh = (2048 + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H);
    int64_t tpw = (a.N + per_bh - 1) / per_bh;
    tpw = ((tpw + 63) / 64) * 64;
    if (tpw < 256) tpw = 256;
    if (a.Dq > 16 || a.Dv > 16) {
        const int nbq = a.Dq / 16, nbv = a.Dv / 16;
        // the operand tables are rebuilt by every workgroup: longer token ranges than for 16 x 16
        if (tpw < 1024) tpw = 1024;
        const size_t lds = (size_t)nbq * nbq * (kD + 1) * 64 * sizeof(uint2) + (size_t)4 * 16 * (a.Dq + 4) * sizeof(float);
        auto kern = dtype == 1 ? triple_out_blocks_kernel<bf16_t> : triple_out_blocks_kernel<f16_t>;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        dim3 grid((unsigned)((a.N + tpw - 1) / tpw) * nbv, a.H, a.B);
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a, (int)tpw);
        return hipGetLastError();
    }
    dim3 grid((unsigned)((a.N + tpw - 1) / tpw), a.H, a.B);
    if (dtype == 1) hipLaunchKernelGGL(triple_out_mfma_kernel<bf16_t>, grid, dim3(256), 0, st, a, (int)tpw);
    else            hipLaunchKernelGGL(triple_out_mfma_kernel<f16_t>, grid, dim3(256), 0, st, a, (int)tpw);
    return hipGetLastError();
}

}  // namespace flare
