// Triple (third-order) linear attention on the matrix cores: bf16 / f16, Dq = Dv = 16.
//
//   state[i,j,k] = (1/N) sum_n f(k1)[n,i] v[n,j] f(k2)[n,k]      (lra/models/backends.py:1289 of the reference)
//   out[n,j]     = sum_{i,k} f(q1)[n,i] state[i,j,k] f(q2)[n,k]  (backends.py:1290)
// For a fixed k both contractions are 16x16x16 products:
//   state[:, :, k] += A_k^T V     with A_k[n,i] = f(k1)[n,i] f(k2)[n,k]           (contraction over 16 tokens)
//   T_k[n,:]        = f(q1)[n,:] state[:, :, k] ;  out[n,:] += T_k[n,:] f(q2)[n,k] (contraction over i)
// so a wave walks 16-token tiles with v_mfma_f32_16x16x16.  Tiles are staged (feature map applied,
// rounded to the element type) in a wave-private LDS tile; operands that need tokens in the
// k-slots come from the LDS transpose read.  No barrier in the token loop and no atomics: a
// workgroup sums its four waves in a fixed order and writes one split partial; the fixed-order
// merge of triple.hip sums the partials.
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

// 4 elements (8 bytes) -> feature map -> repacked; `live` = false gives zeros
template <typename T>
__device__ __forceinline__ uint2 load_feat4(const uint16_t* p, bool live, int fm)
{
    if (!live) return make_uint2(0u, 0u);
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    if (!fm) return raw;
    return make_uint2(Tm<T>::pack2(featf(Tm<T>::lo(raw.x), fm), featf(Tm<T>::hi(raw.x), fm)),
                      Tm<T>::pack2(featf(Tm<T>::lo(raw.y), fm), featf(Tm<T>::hi(raw.y), fm)));
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

// grid (n_splits, H, B); wave w of a workgroup takes the 16-token tiles w, w+4, ... of the split.
template <typename T>
__global__ __launch_bounds__(256) void triple_state_mfma_kernel(TripleArgs a)
{
    using M_ = Tm<T>;
    __shared__ __attribute__((aligned(16))) uint16_t k1s[4][16][kD];
    __shared__ __attribute__((aligned(16))) uint16_t k2s[4][16][kD];
    __shared__ __attribute__((aligned(16))) uint16_t vs[4][16][kD];
    __shared__ __attribute__((aligned(16))) float k2f[4][16][kD];      // f(k2) of the tile in fp32, for the scalar factors
    __shared__ __attribute__((aligned(16))) float red[kD + 1][64][4];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const uint16_t* k1 = (const uint16_t*)a.k1 + b * a.k1s[0] + h * a.k1s[1];
    const uint16_t* k2 = (const uint16_t*)a.k2 + b * a.k2s[0] + h * a.k2s[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    const int n_begin = split * a.tokens_per_split;
    const int n_end = min(a.N, n_begin + a.tokens_per_split);
    const int tok = lane >> 2, piece = (lane & 3) * 4;   // staging: lane = (token, 4 elements)

    f32x4 S[kD], kk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < kD; ++k) S[k] = f32x4{0.f, 0.f, 0.f, 0.f};

    // raw 8-byte pieces of the next tile are fetched while the current one is processed
    auto fetch = [&](int n0, uint2& r1, uint2& r2, uint2& rv) {
        const int n = n0 + tok;
        const bool live = n < n_end;
        r1 = live ? *reinterpret_cast<const uint2*>(k1 + (int64_t)n * a.k1s[2] + piece) : make_uint2(0u, 0u);
        r2 = live ? *reinterpret_cast<const uint2*>(k2 + (int64_t)n * a.k2s[2] + piece) : make_uint2(0u, 0u);
        rv = live ? *reinterpret_cast<const uint2*>(v + (int64_t)n * a.vs[2] + piece) : make_uint2(0u, 0u);
    };
    auto feat4 = [&](uint2 raw, bool live) {
        if (!live) return make_uint2(0u, 0u);
        if (!a.feature_map) return raw;
        return make_uint2(M_::pack2(featf(M_::lo(raw.x), 1), featf(M_::hi(raw.x), 1)),
                          M_::pack2(featf(M_::lo(raw.y), 1), featf(M_::hi(raw.y), 1)));
    };
    uint2 c1, c2, cv, x1, x2, xv;
    fetch(n_begin + w * 16, c1, c2, cv);
    for (int n0 = n_begin + w * 16; n0 < n_end; n0 += 64) {
        const bool live = n0 + tok < n_end;
        fetch(n0 + 64, x1, x2, xv);
        *reinterpret_cast<uint2*>(&k1s[w][tok][piece]) = feat4(c1, live);
        const uint2 f2 = feat4(c2, live);
        *reinterpret_cast<uint2*>(&k2s[w][tok][piece]) = f2;
        *reinterpret_cast<f32x4*>(&k2f[w][tok][piece]) = f32x4{M_::lo(f2.x), M_::hi(f2.x), M_::lo(f2.y), M_::hi(f2.y)};
        *reinterpret_cast<uint2*>(&vs[w][tok][piece]) = live ? cv : make_uint2(0u, 0u);
        c1 = x1; c2 = x2; cv = xv;

        // tokens 4g..4g+3 in the k-slots, lane = feature index c16
        const int tr_row = 4 * g + (c16 >> 2), tr_col = (c16 & 3) * 4;
        const uint2 k1t = tr16(&k1s[w][tr_row][tr_col]);
        const uint2 k2t = tr16(&k2s[w][tr_row][tr_col]);
        const uint2 vt = tr16(&vs[w][tr_row][tr_col]);
        kk = M_::mma16(k1t, k2t, kk);
        const float a0 = M_::lo(k1t.x), a1 = M_::hi(k1t.x), a2 = M_::lo(k1t.y), a3 = M_::hi(k1t.y);
        // f(k2) rows of the lane's four tokens
        f32x4 r[4][4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int c = 0; c < 4; ++c) r[e][c] = *reinterpret_cast<const f32x4*>(&k2f[w][4 * g + e][4 * c]);
#pragma unroll
        for (int k = 0; k < kD; ++k) {
            const int kc = k >> 2, ke = k & 3;
            const uint2 ak = make_uint2(M_::pack2(a0 * r[0][kc][ke], a1 * r[1][kc][ke]), M_::pack2(a2 * r[2][kc][ke], a3 * r[3][kc][ke]));
            S[k] = M_::mma16(ak, vt, S[k]);
        }
    }

    // fixed-order sum of the four waves' accumulators through LDS (wave 1, 2, 3 into wave 0),
    // then one partial per workgroup
    for (int src = 1; src < 4; ++src) {
        __syncthreads();
        if (w == src) {
#pragma unroll
            for (int k = 0; k < kD; ++k) *reinterpret_cast<f32x4*>(&red[k][lane][0]) = S[k];
            *reinterpret_cast<f32x4*>(&red[kD][lane][0]) = kk;
        }
        __syncthreads();
        if (w == 0) {
#pragma unroll
            for (int k = 0; k < kD; ++k) S[k] += *reinterpret_cast<const f32x4*>(&red[k][lane][0]);
            kk += *reinterpret_cast<const f32x4*>(&red[kD][lane][0]);
        }
    }
    if (w != 0) return;
    const size_t per = (size_t)kD * kD * kD + (size_t)kD * kD;
    float* part = a.part + (((size_t)b * a.H + h) * a.n_parts + split) * per;
#pragma unroll
    for (int k = 0; k < kD; ++k)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) part[((size_t)(4 * g + rr) * kD + c16) * kD + k] = S[k][rr];   // [i][j][k]
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) part[(size_t)kD * kD * kD + (size_t)(4 * g + rr) * kD + c16] = kk[rr];   // [i][k']
}

// grid (ceil(N / tokens_per_wg), H, B); each wave walks 16-token tiles of the workgroup's range.
template <typename T>
__global__ __launch_bounds__(256) void triple_out_mfma_kernel(TripleArgs a, int tokens_per_wg)
{
    using M_ = Tm<T>;
    __shared__ __attribute__((aligned(16))) uint16_t q1s[4][16][kD];
    __shared__ __attribute__((aligned(16))) float q2f[4][16][kD];     // f(q2) of the tile in fp32: multiplied as it is

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const uint16_t* q1 = (const uint16_t*)a.q1 + b * a.q1s[0] + h * a.q1s[1];
    const uint16_t* q2 = (const uint16_t*)a.q2 + b * a.q2s[0] + h * a.q2s[1];
    uint16_t* out = (uint16_t*)a.out + b * a.os[0] + h * a.os[1];
    const float* state = a.state + bh * kD * kD * kD;
    const int tok = lane >> 2, piece = (lane & 3) * 4;

    // B operands: sk[k] = state[i = 4g..4g+3][j = c16][k], kkb = kk[i = 4g..4g+3][k' = c16]
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
    // the features of the next tile are fetched while the current one is being worked on
    auto fetch = [&](int n0, uint2& f1, uint2& f2) {
        const int n = n0 + tok;
        const bool live = n < wg_n1;
        f1 = load_feat4<T>(q1 + (int64_t)n * a.q1s[2] + piece, live, a.feature_map);
        f2 = load_feat4<T>(q2 + (int64_t)n * a.q2s[2] + piece, live, a.feature_map);
    };
    uint2 f1 = make_uint2(0u, 0u), f2 = f1;
    if (wg_n0 + w * 16 < wg_n1) fetch(wg_n0 + w * 16, f1, f2);
    for (int n0 = wg_n0 + w * 16; n0 < wg_n1; n0 += 64) {
        *reinterpret_cast<uint2*>(&q1s[w][tok][piece]) = f1;
        *reinterpret_cast<f32x4*>(&q2f[w][tok][piece]) = f32x4{M_::lo(f2.x), M_::hi(f2.x), M_::lo(f2.y), M_::hi(f2.y)};
        if (n0 + 64 < wg_n1) fetch(n0 + 64, f1, f2);

        // A operand: row = token c16, k-slots i = 4g..4g+3
        const uint2 q1a = *reinterpret_cast<const uint2*>(&q1s[w][c16][4 * g]);
        f32x4 r[4][4];       // f(q2)[n = 4g + e][k = 4 c .. 4 c + 3]
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int c = 0; c < 4; ++c) r[e][c] = *reinterpret_cast<const f32x4*>(&q2f[w][4 * g + e][4 * c]);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};   // out[n = 4g + r][j = c16]
#pragma unroll
        for (int k = 0; k < kD; ++k) {
            const f32x4 t = M_::mma16(q1a, sk[k], f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = fmaf(t[e], r[e][k >> 2][k & 3], acc[e]);
        }
        if (a.normalize) {
            // den[n] = sum_k' (f(q1)[n,:] kk[:,k']) f(q2)[n,k'] : k' runs over the 16 lanes of a row group
            const f32x4 wv = M_::mma16(q1a, kkb, f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = acc[e] / row16_sum(wv[e] * q2f[w][4 * g + e][c16]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int nn = n0 + 4 * g + e;
            if (nn < wg_n1) out[(int64_t)nn * a.os[2] + c16] = uint16_t(M_::pack2(acc[e], 0.f) & 0xffffu);
        }
    }
}

}  // namespace

bool triple_mfma_supported(int dtype, int Dq, int Dv) { return (dtype == 1 || dtype == 2) && Dq == 16 && Dv == 16; }

hipError_t launch_triple_state_mfma(const TripleArgs& a, int dtype, hipStream_t st)
{
    dim3 grid(a.n_splits, a.H, a.B);
    if (dtype == 1) hipLaunchKernelGGL(triple_state_mfma_kernel<bf16_t>, grid, dim3(256), 0, st, a);
    else            hipLaunchKernelGGL(triple_state_mfma_kernel<f16_t>, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_triple_out_mfma(const TripleArgs& a, int dtype, hipStream_t st)
{
    // ~8 workgroups per CU over the grid, ranges a multiple of 64 tokens
    const int64_t per_bh = (2048 + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H);
    int64_t tpw = (a.N + per_bh - 1) / per_bh;
    tpw = ((tpw + 63) / 64) * 64;
    if (tpw < 256) tpw = 256;
    dim3 grid((unsigned)((a.N + tpw - 1) / tpw), a.H, a.B);
    if (dtype == 1) hipLaunchKernelGGL(triple_out_mfma_kernel<bf16_t>, grid, dim3(256), 0, st, a, (int)tpw);
    else            hipLaunchKernelGGL(triple_out_mfma_kernel<f16_t>, grid, dim3(256), 0, st, a, (int)tpw);
    return hipGetLastError();
}

}  // namespace flare
