// Causal linear attention on the matrix cores: bf16 / f16 (Dk in {64, 128}, Dv in {32, 64, 128}) and, further down,
// fp32 (Dk in {64, 128}, Dv in {32, 64}).
//
//   y_t = (1/N) sum_{tau <= t} <q_t, k_tau> v_tau        (lra/models/triton/causal_linear.py:317-336)
//
// Same three phases as causal_linear.hip (causal_linear.py:81-137): local states K^T V of token segments, an
// exclusive prefix over the segments, then per segment and 64-token tile  Y = Q S / N + tril(Q K^T) V / N  with the
// running state S advanced tile by tile.  Products run in the element type of the inputs with fp32 accumulation,
// the state is kept in fp32 and handed to the inter-tile product in the element type (scaled by 1/N first, so it
// stays in range), as the reference does for 16-bit inputs (causal_linear.py:262-269).
//
// One workgroup = 4 waves = one segment of one (b,h).  Wave w owns tokens 16 w .. 16 w + 15 of every tile for the
// output and the state rows i = (Dk/4) w .. (Dk/4)(w+1) - 1 for the update.  All products are taken transposed,
//   A^T[tau, t] = sum_i K[tau,i] Q[t,i]        (16x16x32; K rows from LDS, Q rows straight from global memory)
//   Y^T[d, t]  += sum_tau V^T[d,tau] A^T[tau,t] (16x16x32 over two token blocks; the accumulator tiles of A^T, masked and
//                                                packed, are the B operand)
//   Y^T[d, t]  += sum_i S^T[d,i] Q[t,i]         (16x16x32; S^T published in LDS in operand order by its owners)
//   S[i, d]    += sum_tau K^T[i,tau] V[tau,d]   (16x16x32; both operands by transposed LDS reads)
// so that a lane ends up with four consecutive channels of one token's output row.
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

template <typename T> struct Ml;
template <> struct Ml<bf16_t> {
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
};
template <> struct Ml<f16_t> {
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
};

// ds_read_b64_tr_b16 of a 16-bit [row][column] tile: the lane at (g, c16) passes the address of row 4g + (c16 >> 2),
// column 4 (c16 & 3) of a 16 x 16 block and receives the block's elements (row 4g + e, column c16), e = 0..3:
// the operand of a product over the rows, for whichever side the columns are.
__device__ __forceinline__ uint2 tr16(const void* lds_addr)
{
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    asm volatile("" ::: "memory");
    const s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)lds_addr);
    asm volatile("" ::: "memory");
    return __builtin_bit_cast(uint2, r);
}

constexpr int kTile = 64;   // tokens per tile
constexpr int kPad = 8;     // 16-bit elements of padding per LDS row (the rows of a transposed read fall into different banks)

template <int DK, int DV, bool STATE_ONLY>
constexpr size_t lds_bytes()
{
    return (size_t)kTile * (DK + kPad + DV + kPad) * 2 + (STATE_ONLY ? 0 : (size_t)(DV / 16) * (DK / 32) * 64 * 16);
}

template <typename T, int DK, int DV, bool STATE_ONLY>
__global__ __launch_bounds__(256, 2) void causal_linear_mfma_kernel(CausalLinearArgs a)
{
    constexpr int KD = DK / 32, IT = DK / 16, DT = DV / 16;
    constexpr int ITW = IT / 4;                      // 16-row tiles of the state per wave
    constexpr int KS = DK + kPad, VS = DV + kPad;    // LDS row strides in elements
    constexpr int KPT = kTile * (DK / 8) / 256;      // 16-byte chunks of a K tile per thread
    constexpr int VPT = kTile * (DV / 8) / 256;      // and of a V tile
    static_assert(IT % 4 == 0 && KPT >= 1 && VPT >= 1, "Dk in {64, 128}, Dv in {32, 64, 128}");
    using M_ = Ml<T>;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t* kt = reinterpret_cast<uint16_t*>(smem);            // [64][KS]
    uint16_t* vt = kt + kTile * KS;                               // [64][VS]
    u32x4* sop = reinterpret_cast<u32x4*>(vt + kTile * VS);       // [DT][KD][64]: S^T / N as A operands

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int seg = blockIdx.x, bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const uint16_t* q = (const uint16_t*)a.q + b * a.qs[0] + h * a.qs[1];
    const uint16_t* k = (const uint16_t*)a.k + b * a.ks[0] + h * a.ks[1];
    const uint16_t* v = (const uint16_t*)a.v + b * a.vs[0] + h * a.vs[1];
    uint16_t* y = (uint16_t*)a.y + b * a.ys[0] + h * a.ys[1];
    float* slot = a.states + ((int64_t)bh * a.n_segs + seg) * DK * DV;
    const int n_lo = seg * a.seg_len, n_hi = min(a.N, n_lo + a.seg_len);
    const int tiles = (n_hi - n_lo + kTile - 1) / kTile;

    // the wave's rows of the state: tile (itw, dt) holds S[16 (w ITW + itw) + 4g + r][16 dt + c16]
    f32x4 U[ITW][DT];
#pragma unroll
    for (int itw = 0; itw < ITW; ++itw)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                U[itw][dt][r] = STATE_ONLY ? 0.f : slot[(int64_t)(16 * (w * ITW + itw) + 4 * g + r) * DV + 16 * dt + c16];

    // one register set: the next tile is requested at the top of an iteration and handed to LDS at its bottom.
    // Rows past the end of the segment repeat its last row (no branch around a load) and are staged as zeros.
    u32x4 kr[KPT], vr[VPT], qn[KD], qc[KD];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int c = tid + i * 256, tok = c / (DK / 8), ch = c % (DK / 8);
            kr[i] = *reinterpret_cast<const u32x4*>(k + (int64_t)min(n0 + tok, n_hi - 1) * a.ks[2] + ch * 8);
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = tid + i * 256, tok = c / (DV / 8), ch = c % (DV / 8);
            vr[i] = *reinterpret_cast<const u32x4*>(v + (int64_t)min(n0 + tok, n_hi - 1) * a.vs[2] + ch * 8);
        }
        if constexpr (!STATE_ONLY) {
            const int n = min(n0 + 16 * w + c16, n_hi - 1);
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) qn[kd] = *reinterpret_cast<const u32x4*>(q + (int64_t)n * a.qs[2] + 32 * kd + 8 * g);
        }
    };
    auto stage = [&](int n0) {
        const u32x4 z4 = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int c = tid + i * 256, tok = c / (DK / 8), ch = c % (DK / 8);
            *reinterpret_cast<u32x4*>(kt + tok * KS + ch * 8) = n0 + tok < n_hi ? kr[i] : z4;
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = tid + i * 256, tok = c / (DV / 8), ch = c % (DV / 8);
            *reinterpret_cast<u32x4*>(vt + tok * VS + ch * 8) = n0 + tok < n_hi ? vr[i] : z4;
        }
    };
    // S^T / N in the operand order of the inter-tile product: the entry of lane (gl, cl) of tile (dt, kd) holds
    // S[32 kd + 8 gl + e][16 dt + cl], e = 0..7.  The owner of S[16 it + 4g + r][16 dt + c16] writes its four rows
    // as 8 bytes of the entry of lane (2 (it & 1) + (g >> 1), c16), half g & 1.
    auto publish = [&]() {
#pragma unroll
        for (int itw = 0; itw < ITW; ++itw) {
            const int it = w * ITW + itw, kd = it >> 1, gl = 2 * (it & 1) + (g >> 1);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const f32x4 u = U[itw][dt] * a.inv_n;
                uint8_t* e = reinterpret_cast<uint8_t*>(sop + (dt * KD + kd) * 64 + gl * 16 + c16) + 8 * (g & 1);
                *reinterpret_cast<uint2*>(e) = make_uint2(M_::pack2(u[0], u[1]), M_::pack2(u[2], u[3]));
            }
        }
    };
    // two 16-token blocks as one operand of a 32-deep product: k-slots 8g + e = token 4g + e of block bl for e < 4,
    // of block bl + 1 for e >= 4 (any order of the contraction index will do as long as both operands agree)
    auto tr32 = [&](const uint16_t* tile, int stride, int bl, int col) {
        const uint2 lo = tr16(tile + (16 * bl + 4 * g + (c16 >> 2)) * stride + col + 4 * (c16 & 3));
        const uint2 hi = tr16(tile + (16 * bl + 16 + 4 * g + (c16 >> 2)) * stride + col + 4 * (c16 & 3));
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    };
    // S += K^T V over the 64 tokens of the staged tile, for the wave's rows of S
    auto update = [&]() {
#pragma unroll
        for (int bl = 0; bl < 4; bl += 2) {
            u32x4 vop[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vop[dt] = tr32(vt, VS, bl, 16 * dt);
#pragma unroll
            for (int itw = 0; itw < ITW; ++itw) {
                const u32x4 kop = tr32(kt, KS, bl, 16 * (w * ITW + itw));
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) U[itw][dt] = M_::mma32(kop, vop[dt], U[itw][dt]);
            }
        }
    };

    if (tiles > 0) {
        fetch(n_lo);
        stage(n_lo);
        if constexpr (!STATE_ONLY) {
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) qc[kd] = qn[kd];
            publish();
        }
    }
    __syncthreads();

    const f32x4 zf = {0.f, 0.f, 0.f, 0.f};
    int n0 = n_lo;
    for (int t = 0; t < tiles; ++t, n0 += kTile) {
        fetch(n0 + kTile);      // unconditional: past the end the last rows are read again and never used

        if constexpr (!STATE_ONLY) {
            // this tile: tril(Q K^T) V, the token blocks up to the wave's own
            f32x4 yacc[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) yacc[dt] = zf;
            // A^T of a block: lane = column t = c16, rows tau = 4g + r; the diagonal block keeps tau <= t
            auto block_scores = [&](int bl) {
                f32x4 s = zf;
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) {
                    const u32x4 ka = *reinterpret_cast<const u32x4*>(kt + (16 * bl + c16) * KS + 32 * kd + 8 * g);
                    s = M_::mma32(ka, qc[kd], s);
                }
                if (bl == w) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) s[r] = 4 * g + r <= c16 ? s[r] : 0.f;
                }
                return make_uint2(M_::pack2(s[0], s[1]), M_::pack2(s[2], s[3]));
            };
#pragma unroll
            for (int bl = 0; bl < 4; bl += 2) {
                if (bl > w) break;      // uniform over the wave
                const uint2 p0 = block_scores(bl);
                uint2 p1 = make_uint2(0u, 0u);
                if (bl + 1 <= w) p1 = block_scores(bl + 1);
                const u32x4 pb = {p0.x, p0.y, p1.x, p1.y};
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) yacc[dt] = M_::mma32(tr32(vt, VS, bl, 16 * dt), pb, yacc[dt]);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) yacc[dt] *= a.inv_n;
            // earlier tiles and segments: Q S / N
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) yacc[dt] = M_::mma32(sop[(dt * KD + kd) * 64 + lane], qc[kd], yacc[dt]);
            // The next tile's rows are waited for here, before the stores: loads and stores complete in order on one
            // counter and the stores sit under a per-lane condition, so a wait behind them would wait for all of them.
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
            const int n = n0 + 16 * w + c16;
            if (n < n_hi) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    *reinterpret_cast<uint2*>(y + (int64_t)n * a.ys[2] + 16 * dt + 4 * g) =
                        make_uint2(M_::pack2(yacc[dt][0], yacc[dt][1]), M_::pack2(yacc[dt][2], yacc[dt][3]));
            }
        }

        update();
        __syncthreads();        // everyone is done with this tile's K, V and state operands
        stage(n0 + kTile);
        if constexpr (!STATE_ONLY) {
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) qc[kd] = qn[kd];
            publish();
        }
        __syncthreads();
    }

    if constexpr (STATE_ONLY) {
#pragma unroll
        for (int itw = 0; itw < ITW; ++itw)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    slot[(int64_t)(16 * (w * ITW + itw) + 4 * g + r) * DV + 16 * dt + c16] = U[itw][dt][r];
    }
}

// ---- fp32 inputs: the same scheme on v_mfma_f32_16x16x4_f32 ------------------------------------------------------
// A: lane (row c16, k = g) one float, B: lane (column c16, k = g) one float, accumulators as above.  A product over Dk
// takes Dk/4 instructions; the k-slot of lane group g in instruction j is feature g Dk/4 + j, so that a lane's share of a
// Q or K row is contiguous (16-byte loads).  An accumulator tile of A^T (lane = token t, registers = tokens tau = 4g + r)
// is the B operand of four instructions of the next product, register r for the instruction whose k-slots are 4g + r.
template <int DK, int DV, bool STATE_ONLY>
constexpr size_t lds_bytes_f32()
{
    return (size_t)kTile * (DK + 4 + DV + 4) * 4 + (STATE_ONLY ? 0 : (size_t)DV * DK * 4);
}

template <int DK, int DV, bool STATE_ONLY>
__global__ __launch_bounds__(256, 2) void causal_linear_f32_kernel(CausalLinearArgs a)
{
    constexpr int QL = DK / 4;                       // features per lane group
    constexpr int IT = DK / 16, DT = DV / 16, ITW = IT / 4;
    constexpr int KS = DK + 4, VS = DV + 4;          // LDS row strides in floats
    constexpr int KPT = kTile * (DK / 4) / 256, VPT = kTile * (DV / 4) / 256;
    static_assert(IT % 4 == 0 && VPT >= 1, "Dk in {64, 128}, Dv a multiple of 16 from 16");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float* kt = reinterpret_cast<float*>(smem);      // [64][KS]
    float* vt = kt + kTile * KS;                     // [64][VS]
    float* sop = vt + kTile * VS;                    // [DT][QL][64]: S^T / N as A operands of the inter-tile product

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int seg = blockIdx.x, bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const float* q = (const float*)a.q + b * a.qs[0] + h * a.qs[1];
    const float* k = (const float*)a.k + b * a.ks[0] + h * a.ks[1];
    const float* v = (const float*)a.v + b * a.vs[0] + h * a.vs[1];
    float* y = (float*)a.y + b * a.ys[0] + h * a.ys[1];
    float* slot = a.states + ((int64_t)bh * a.n_segs + seg) * DK * DV;
    const int n_lo = seg * a.seg_len, n_hi = min(a.N, n_lo + a.seg_len);
    const int tiles = (n_hi - n_lo + kTile - 1) / kTile;

    f32x4 U[ITW][DT];
#pragma unroll
    for (int itw = 0; itw < ITW; ++itw)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                U[itw][dt][r] = STATE_ONLY ? 0.f : slot[(int64_t)(16 * (w * ITW + itw) + 4 * g + r) * DV + 16 * dt + c16];

    f32x4 kr[KPT], vr[VPT], qn[QL / 4], qc[QL / 4];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int c = tid + i * 256, tok = c / (DK / 4), ch = c % (DK / 4);
            kr[i] = *reinterpret_cast<const f32x4*>(k + (int64_t)min(n0 + tok, n_hi - 1) * a.ks[2] + ch * 4);
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = tid + i * 256, tok = c / (DV / 4), ch = c % (DV / 4);
            vr[i] = *reinterpret_cast<const f32x4*>(v + (int64_t)min(n0 + tok, n_hi - 1) * a.vs[2] + ch * 4);
        }
        if constexpr (!STATE_ONLY) {
            const int n = min(n0 + 16 * w + c16, n_hi - 1);
#pragma unroll
            for (int j = 0; j < QL / 4; ++j) qn[j] = *reinterpret_cast<const f32x4*>(q + (int64_t)n * a.qs[2] + g * QL + 4 * j);
        }
    };
    auto stage = [&](int n0) {
        const f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int c = tid + i * 256, tok = c / (DK / 4), ch = c % (DK / 4);
            *reinterpret_cast<f32x4*>(kt + tok * KS + ch * 4) = n0 + tok < n_hi ? kr[i] : z4;
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = tid + i * 256, tok = c / (DV / 4), ch = c % (DV / 4);
            *reinterpret_cast<f32x4*>(vt + tok * VS + ch * 4) = n0 + tok < n_hi ? vr[i] : z4;
        }
    };
    // entry (dt, j, lane (gl, cl)) = S[gl QL + j][16 dt + cl] / N; the owner of S[i][16 dt + c16] writes it there
    auto publish = [&]() {
#pragma unroll
        for (int itw = 0; itw < ITW; ++itw)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * (w * ITW + itw) + 4 * g + r;
                    sop[(dt * QL + i % QL) * 64 + (i / QL) * 16 + c16] = U[itw][dt][r] * a.inv_n;
                }
    };
    auto update = [&]() {
#pragma unroll
        for (int m = 0; m < kTile / 4; ++m) {       // tokens 4m + g
            float vop[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vop[dt] = vt[(4 * m + g) * VS + 16 * dt + c16];
#pragma unroll
            for (int itw = 0; itw < ITW; ++itw) {
                const float kop = kt[(4 * m + g) * KS + 16 * (w * ITW + itw) + c16];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) U[itw][dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(kop, vop[dt], U[itw][dt], 0, 0, 0);
            }
        }
    };

    if (tiles > 0) {
        fetch(n_lo);
        stage(n_lo);
        if constexpr (!STATE_ONLY) {
#pragma unroll
            for (int j = 0; j < QL / 4; ++j) qc[j] = qn[j];
            publish();
        }
    }
    __syncthreads();

    const f32x4 zf = {0.f, 0.f, 0.f, 0.f};
    int n0 = n_lo;
    for (int t = 0; t < tiles; ++t, n0 += kTile) {
        fetch(n0 + kTile);

        if constexpr (!STATE_ONLY) {
            f32x4 yacc[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) yacc[dt] = zf;
#pragma unroll
            for (int bl = 0; bl < 4; ++bl) {
                if (bl > w) break;      // uniform over the wave
                f32x4 s = zf;
#pragma unroll
                for (int j4 = 0; j4 < QL / 4; ++j4) {
                    const f32x4 ka = *reinterpret_cast<const f32x4*>(kt + (16 * bl + c16) * KS + g * QL + 4 * j4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) s = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[e], qc[j4][e], s, 0, 0, 0);
                }
                if (bl == w) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) s[r] = 4 * g + r <= c16 ? s[r] : 0.f;
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        yacc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vt[(16 * bl + 4 * g + r) * VS + 16 * dt + c16], s[r], yacc[dt], 0, 0, 0);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) yacc[dt] *= a.inv_n;
#pragma unroll
            for (int j4 = 0; j4 < QL / 4; ++j4)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        yacc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sop[(dt * QL + 4 * j4 + e) * 64 + lane], qc[j4][e], yacc[dt], 0, 0, 0);
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the next tile's rows, before the stores (see the 16-bit kernel)
            const int n = n0 + 16 * w + c16;
            if (n < n_hi) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(y + (int64_t)n * a.ys[2] + 16 * dt + 4 * g) = yacc[dt];
            }
        }

        update();
        __syncthreads();
        stage(n0 + kTile);
        if constexpr (!STATE_ONLY) {
#pragma unroll
            for (int j = 0; j < QL / 4; ++j) qc[j] = qn[j];
            publish();
        }
        __syncthreads();
    }

    if constexpr (STATE_ONLY) {
#pragma unroll
        for (int itw = 0; itw < ITW; ++itw)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    slot[(int64_t)(16 * (w * ITW + itw) + 4 * g + r) * DV + 16 * dt + c16] = U[itw][dt][r];
    }
}

template <int DK, int DV>
hipError_t launch_f32_dd(const CausalLinearArgs& a, hipStream_t st)
{
    const int BH = a.B * a.H;
    auto state_k = causal_linear_f32_kernel<DK, DV, true>;
    auto out_k = causal_linear_f32_kernel<DK, DV, false>;
    constexpr size_t lds_s = lds_bytes_f32<DK, DV, true>(), lds_o = lds_bytes_f32<DK, DV, false>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(state_k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_s);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(out_k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_o);
    if (e != hipSuccess) return e;
    if (a.n_segs > 1) hipLaunchKernelGGL(state_k, dim3(a.n_segs - 1, BH), dim3(256), lds_s, st, a);
    e = launch_causal_linear_prefix(a, st);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(out_k, dim3(a.n_segs, BH), dim3(256), lds_o, st, a);
    return hipGetLastError();
}

hipError_t launch_f32(const CausalLinearArgs& a, hipStream_t st)
{
    if (a.Dk == 64 && a.Dv == 32) return launch_f32_dd<64, 32>(a, st);
    if (a.Dk == 64 && a.Dv == 64) return launch_f32_dd<64, 64>(a, st);
    if (a.Dk == 128 && a.Dv == 32) return launch_f32_dd<128, 32>(a, st);
    if (a.Dk == 128 && a.Dv == 64) return launch_f32_dd<128, 64>(a, st);
    return hipErrorInvalidValue;
}

template <typename T, int DK, int DV>
hipError_t launch_dd(const CausalLinearArgs& a, hipStream_t st)
{
    const int BH = a.B * a.H;
    auto state_k = causal_linear_mfma_kernel<T, DK, DV, true>;
    auto out_k = causal_linear_mfma_kernel<T, DK, DV, false>;
    constexpr size_t lds_s = lds_bytes<DK, DV, true>(), lds_o = lds_bytes<DK, DV, false>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(state_k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_s);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(out_k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_o);
    if (e != hipSuccess) return e;
    if (a.n_segs > 1) hipLaunchKernelGGL(state_k, dim3(a.n_segs - 1, BH), dim3(256), lds_s, st, a);
    e = launch_causal_linear_prefix(a, st);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(out_k, dim3(a.n_segs, BH), dim3(256), lds_o, st, a);
    return hipGetLastError();
}

template <typename T, int DK>
hipError_t launch_d(const CausalLinearArgs& a, hipStream_t st)
{
    switch (a.Dv) {
        case 32:  return launch_dd<T, DK, 32>(a, st);
        case 64:  return launch_dd<T, DK, 64>(a, st);
        case 128: return launch_dd<T, DK, 128>(a, st);
        default:  return hipErrorInvalidValue;
    }
}

template <typename T>
hipError_t launch_t(const CausalLinearArgs& a, hipStream_t st)
{
    if (a.Dk == 64) return launch_d<T, 64>(a, st);
    if (a.Dk == 128) return launch_d<T, 128>(a, st);
    return hipErrorInvalidValue;
}

}  // namespace

bool causal_linear_mfma_supported(int dtype, int Dk, int Dv)
{
    if (dtype == 0) return (Dk == 64 || Dk == 128) && (Dv == 32 || Dv == 64);
    return (dtype == 1 || dtype == 2) && (Dk == 64 || Dk == 128) && (Dv == 32 || Dv == 64 || Dv == 128);
}

hipError_t launch_causal_linear_mfma(const CausalLinearArgs& a, int dtype, hipStream_t st)
{
    if (dtype == 0) return launch_f32(a, st);
    return dtype == 1 ? launch_t<bf16_t>(a, st) : launch_t<f16_t>(a, st);
}

}  // namespace flare
