// Fused token-wise MLP stack on the matrix cores (bf16 / f16 weights, C in {32, 64, 128}).
//
// One launch evaluates, per token, what pdebench/models/flare.py of the reference spells as
// separate torch layers: an optional LayerNorm / RMSNorm (FLAREBlock.forward :204-215), a chain of
// C x C Linear layers each optionally followed by the activation and optionally added to the
// running stream (ResidualMLP.forward :45-59; a single Linear is the chain of length one), and an
// optional outer residual.  Layer l:  t = W_l s + b_l;  t = act(t) if bit l of act_mask;
// s = s + t if bit l of add_mask else t.   Output = res + s  (res may be absent).
// Expanding mode (a.expand): the two-layer MLP with hidden width E*C, y = W2 act(W1 n + b1) + b2, as E pairs of
// C x C tiles: h_j = act(W1[j] n + b1[j]) from the packed input n, then s += W2[:, j] h_j, the hidden chunk h_j
// never leaving the registers (tiles come as L = 2E "layers": W1[0], W2[:,0], W1[1], W2[:,1], ...).
// Lifting mode (a.in_dim > 0): the rows of x have only in_dim <= 4 features (coordinates and a field value, say)
// and a first layer C x in_dim, evaluated with in_dim multiply-adds per output on the vector ALU, produces the
// stream that the C x C chain continues from (ResidualMLP(in_dim, C, C, ...), the models' input projection).
// Projecting mode (a.out_dim > 0): the last tile has only out_dim <= 4 real rows (the rest are zero) and only those
// outputs are stored, y rows being out_dim wide (ResidualMLP(C, C, out_dim, ...), the models' output projection).
// Head-padded rows (a.x_head / a.y_head > 0, an instance of their own): the C channels of a row are H heads of fewer
// than 16 channels and each head occupies 16 columns, the layout the mixer's matrix-core kernels read and write
// for narrow heads -- the projections write it and the output projection reads it, so nothing is copied between.
//
// Layout.  The product is taken transposed, S'^T = W S^T, with v_mfma_f32_16x16x32: A = W tile
// (lane = output row, 8 consecutive input features per lane), B = S^T (lane = token c16, k-slots =
// input features), D: lane = token, registers = 4 output rows.  Lane (c16, g) of stream tile ft
// holds features 16 ft + 4 g + r (r = 0..3) of token c16.  Therefore
//   * x, res and y move as 4-element runs per lane; the 4 lanes of a token cover 16 consecutive
//     features per instruction (64 contiguous bytes of fp32 per row),
//   * the accumulators of one layer, packed to 16 bits in place, ARE the B operands of the next
//     layer: a contraction may visit its index in any order, so k-slot e of step ks in lane g is
//     simply feature 32 ks + 16 (e/4) + 4 g + e%4, and the stream never leaves the registers
//     between layers (fp32 on the residual path),
//   * the weights are staged into LDS with their columns in that slot order, so the A operand of
//     step ks is one 16-byte read at column position 32 ks + 8 g.
// Weights live in LDS, shared by the WAVES waves of a workgroup, each of which owns 16*TW tokens
// per pass.  When all L layers fit they are staged once and the token loop has no barrier at all;
// otherwise two slots form a ring: the next layer's weights are fetched into registers before the
// products of the current layer and written to the free slot after them (one barrier per layer).
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

template <typename T> struct Mm;
template <> struct Mm<bf16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
};
template <> struct Mm<f16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
};

// four consecutive elements of a row of element type dt (0 f32, 1 bf16, 2 f16) as fp32
__device__ __forceinline__ f32x4 load4(const void* base, int64_t elem, int dt)
{
    if (dt == 0) return *reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem);
    const uint2 r = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + elem);
    if (dt == 1)
        return f32x4{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                     __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u)};
    const f16x2 lo = __builtin_bit_cast(f16x2, r.x), hi = __builtin_bit_cast(f16x2, r.y);
    return f32x4{(float)lo[0], (float)lo[1], (float)hi[0], (float)hi[1]};
}

__device__ __forceinline__ void store4(void* base, int64_t elem, int dt, f32x4 v)
{
    if (dt == 0) {
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + elem) = v;
    } else if (dt == 1) {
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + elem) =
            make_uint2(Mm<bf16_t>::pack2(v[0], v[1]), Mm<bf16_t>::pack2(v[2], v[3]));
    } else {
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + elem) =
            make_uint2(Mm<f16_t>::pack2(v[0], v[1]), Mm<f16_t>::pack2(v[2], v[3]));
    }
}

__device__ __forceinline__ float xg_sum(float v)   // sum over the 4 lane groups that share a token
{
    v = sum_xor16(v);
    v = sum_xor32(v);
    return v;
}

// tanh-GELU (torch's approximate='tanh') = x * sigmoid(2 u), u = sqrt(2/pi) (x + 0.044715 x^3); the gate is the sigmoid
__device__ __forceinline__ float gelu_gate(float x)
{
    const float t = x * (2.3022081f + 0.10294324f * x * x);      // 2 u log2(e)
    return __builtin_amdgcn_rcpf(1.f + fast_exp2(-t));
}
__device__ __forceinline__ float silu_gate(float x)
{
    return __builtin_amdgcn_rcpf(1.f + fast_exp2(-kLog2e * x));
}

// MODE: 0 the C x C chain, 1 the expanding two-layer MLP, 2 the chain with a narrow first input and/or last output,
// 3 the chain with head-padded rows on either end
template <typename T, int C, int TW, int WAVES, int MODE>
__global__ __launch_bounds__(64 * WAVES, (512 / (64 * WAVES) > 0 ? 512 / (64 * WAVES) : 1)) void mlp_mfma_kernel(MlpArgs a, int resident)
{
    constexpr int NT = 64 * WAVES;
    constexpr int NCH = (C * C / 8 + NT - 1) / NT;   // 16-byte weight chunks per thread and layer
    constexpr int FT = C / 16;        // feature tiles of the stream
    constexpr int KS = C / 32;        // k-steps of one layer
    constexpr int RS = C * 2;         // LDS row stride in bytes; no padding: the 16-byte chunks of a row are
    constexpr int WBUF = C * RS;      // XOR-swizzled with the row number so that 16 rows read 16 different bank groups
    constexpr int CPR = C / 8;        // 16-byte chunks per row
    constexpr int SWS = CPR == 16 ? 0 : CPR == 8 ? 1 : 2;   // swizzle key of row r: ((r & 15) >> SWS), below CPR
    constexpr int TOKW = 16 * TW;     // tokens per wave and pass
    using M_ = Mm<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;

    u32x4 wreg[NCH];
    auto fetch = [&](int layer) {
        const uint16_t* wl = a.w + (size_t)layer * C * C;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * NT;
            if (c < C * C / 8) wreg[i] = *reinterpret_cast<const u32x4*>(wl + (c / (C / 8)) * C + (c % (C / 8)) * 8);
        }
    };
    auto put = [&](int slot) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * NT;
            if (c < C * C / 8) {
                const int row = c / (C / 8), ch = c % (C / 8);
                // features 8 ch .. 8 ch + 3 belong to k-step ch / 4, half (ch % 4) / 2, lane group 2 (ch % 2);
                // features 8 ch + 4 .. + 7 to the next lane group.  Position = 32 ks + 8 g + 4 half.
                // In 16-byte chunks: chunk 4 ks + 2 (ch % 2) and the one after it, 8-byte half (ch % 4) / 2.
                const int chunk = 4 * (ch >> 2) + 2 * (ch & 1), half = (ch & 3) >> 1;
                const int key = (row & 15) >> SWS;
                uint8_t* dst = smem + slot * WBUF + row * RS + half * 8;
                *reinterpret_cast<uint2*>(dst + ((chunk ^ key) << 4)) = make_uint2(wreg[i][0], wreg[i][1]);
                *reinterpret_cast<uint2*>(dst + (((chunk + 1) ^ key) << 4)) = make_uint2(wreg[i][2], wreg[i][3]);
            }
        }
    };

    // Parameter vectors are read without a branch (a branch per feature tile keeps the compiler from issuing the
    // loads ahead of where they are used): a missing vector reads the weights instead, any mapped memory will do,
    // and is replaced by zeros.
    const bool has_bias = a.bias != nullptr, has_beta = a.beta != nullptr;
    const float* bias0 = has_bias ? a.bias : reinterpret_cast<const float*>(a.w);
    const float* beta0 = has_beta ? a.beta : reinterpret_cast<const float*>(a.w);
    auto vec4 = [](const float* p, bool have) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(p);
        return have ? v : f32x4{0.f, 0.f, 0.f, 0.f};
    };

    int woff[KS];     // byte offset of this lane's chunk of k-step ks inside its weight row (swizzled)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) woff[ks] = ((4 * ks + g) ^ (c16 >> SWS)) << 4;

    int lcount = 0;   // ring mode: layers done by this workgroup; its parity names the slot in use
    if (resident) {
        for (int l = 0; l < a.L; ++l) {
            fetch(l);
            put(l);
        }
    } else {
        fetch(0);
        put(0);
    }
    __syncthreads();

    const int64_t nblk = ((int64_t)a.T + WAVES * TOKW - 1) / (WAVES * TOKW);
    for (int64_t blk = blockIdx.x; blk < nblk; blk += gridDim.x) {
        int64_t tok[TW];
        bool live[TW];
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
            const int64_t t = blk * (WAVES * TOKW) + w * TOKW + tw * 16 + c16;
            live[tw] = t < a.T;
            tok[tw] = live[tw] ? t : a.T - 1;
        }

        // the stream: lane (c16, g) holds features 16 ft + 4 g + r of token c16 of each tile
        f32x4 xs[FT][TW];
        if (MODE == 2 && a.in_dim > 0) {
            // lifting layer: s[f] = act(b_in[f] + sum_i w_in[f][i] x[i]) from the token's few input features
            float xin[TW][4];
#pragma unroll
            for (int tw = 0; tw < TW; ++tw)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v = 0.f;
                    if (i < a.in_dim) {
                        const int64_t e = tok[tw] * a.xs + i;
                        v = a.x_dtype == 0 ? static_cast<const float*>(a.x)[e]
                          : a.x_dtype == 1 ? __uint_as_float(uint32_t(static_cast<const uint16_t*>(a.x)[e]) << 16)
                                           : (float)static_cast<const _Float16*>(a.x)[e];
                    }
                    xin[tw][i] = v;
                }
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 b4 = *reinterpret_cast<const f32x4*>(a.b_in + 16 * ft + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const f32x4 wr = *reinterpret_cast<const f32x4*>(a.w_in + (16 * ft + 4 * g + r) * 4);
#pragma unroll
                    for (int tw = 0; tw < TW; ++tw) {
                        float t = b4[r];
#pragma unroll
                        for (int i = 0; i < 4; ++i) t = fmaf(wr[i], xin[tw][i], t);
                        if (a.in_act) t *= a.act == 0 ? gelu_gate(t) : silu_gate(t);
                        xs[ft][tw][r] = t;
                    }
                }
            }
        } else if (MODE == 3 && a.x_head > 0) {
            // head-padded rows: channel f = 16 ft + 4 g of the row sits at column 16 (f / x_head) + f % x_head,
            // which is ft * 32 + 8 g - 4 (g & 1) for heads of 8 and ft * 64 + 16 g for heads of 4
            const int cf = a.x_head == 8 ? 32 : 64, c0 = a.x_head == 8 ? 8 * g - 4 * (g & 1) : 16 * g;
#pragma unroll
            for (int tw = 0; tw < TW; ++tw)
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) xs[ft][tw] = load4(a.x, tok[tw] * a.xs + ft * cf + c0, a.x_dtype);
        } else {
#pragma unroll
            for (int tw = 0; tw < TW; ++tw)
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) xs[ft][tw] = load4(a.x, tok[tw] * a.xs + 16 * ft + 4 * g, a.x_dtype);
        }

        if (a.norm != 0) {
#pragma unroll
            for (int tw = 0; tw < TW; ++tw) {
                // the row sum is taken for both norms and dropped for RMSNorm: straight-line code (with the sum
                // under a branch, the one-token-tile instances of this kernel came out wrong for RMSNorm)
                float s = 0.f;
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) s += xs[ft][tw][0] + xs[ft][tw][1] + xs[ft][tw][2] + xs[ft][tw][3];
                const float rowmean = xg_sum(s) * (1.f / C);
                const float mean = a.norm == 1 ? rowmean : 0.f;
                float ss = 0.f;
#pragma unroll
                for (int ft = 0; ft < FT; ++ft)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float d = xs[ft][tw][r] - mean;
                        ss = fmaf(d, d, ss);
                    }
                const float rstd = rsqrtf(xg_sum(ss) * (1.f / C) + a.eps);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    const f32x4 gm = *reinterpret_cast<const f32x4*>(a.gamma + 16 * ft + 4 * g);
                    const f32x4 bt = vec4(beta0 + 16 * ft + 4 * g, has_beta);
#pragma unroll
                    for (int r = 0; r < 4; ++r) xs[ft][tw][r] = (xs[ft][tw][r] - mean) * rstd * gm[r] + bt[r];
                }
            }
        }

        if constexpr (MODE == 1) {
            // n = the (normalised) input, packed once; the stream restarts at zero and collects the second products
            u32x4 xb0[KS][TW], hb[KS][TW];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int tw = 0; tw < TW; ++tw) {
                    const f32x4 lo = xs[2 * ks][tw], hi = xs[2 * ks + 1][tw];
                    xb0[ks][tw] = u32x4{M_::pack2(lo[0], lo[1]), M_::pack2(lo[2], lo[3]),
                                        M_::pack2(hi[0], hi[1]), M_::pack2(hi[2], hi[3])};
                    hb[ks][tw] = xb0[ks][tw];
                }
#pragma unroll
            for (int ft = 0; ft < FT; ++ft)
#pragma unroll
                for (int tw = 0; tw < TW; ++tw) xs[ft][tw] = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int l = 0; l < a.L; ++l, ++lcount) {
                const int slot = resident ? l : (lcount & 1);
                if (!resident) fetch(l + 1 < a.L ? l + 1 : 0);
                const uint8_t* wb = smem + slot * WBUF + c16 * RS;
                const float* bl = bias0 + (size_t)l * C + 4 * g;
                if (!(l & 1)) {
                    // h = act(W1[j] n + b1[j]): tile ft of h is half (ft & 1) of k-step ft / 2 of the next product
                    auto first = [&](auto act_c) {
                        constexpr int ACT = decltype(act_c)::value;
                        // bias rows requested two feature tiles ahead, as in the chain below
                        f32x4 bias_q[2];
#pragma unroll
                        for (int i = 0; i < 2; ++i) bias_q[i] = vec4(bl + 16 * (i < FT ? i : 0), has_bias);
#pragma unroll
                        for (int ft = 0; ft < FT; ++ft) {
                            const f32x4 bias = bias_q[ft & 1];
                            if (ft + 2 < FT) bias_q[ft & 1] = vec4(bl + 16 * (ft + 2), has_bias);
                            f32x4 acc[TW];
#pragma unroll
                            for (int tw = 0; tw < TW; ++tw) acc[tw] = bias;
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks) {
                                const u32x4 wa = *reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[ks]);
#pragma unroll
                                for (int tw = 0; tw < TW; ++tw) acc[tw] = M_::mma(wa, xb0[ks][tw], acc[tw]);
                            }
#pragma unroll
                            for (int tw = 0; tw < TW; ++tw) {
                                float t[4];
#pragma unroll
                                for (int r = 0; r < 4; ++r)
                                    t[r] = ACT == 0 ? acc[tw][r] : acc[tw][r] * (ACT == 1 ? gelu_gate(acc[tw][r]) : silu_gate(acc[tw][r]));
                                hb[ft >> 1][tw][2 * (ft & 1)] = M_::pack2(t[0], t[1]);
                                hb[ft >> 1][tw][2 * (ft & 1) + 1] = M_::pack2(t[2], t[3]);
                            }
                        }
                    };
                    if (!((a.act_mask >> l) & 1u)) first(std::integral_constant<int, 0>{});
                    else if (a.act == 0) first(std::integral_constant<int, 1>{});
                    else first(std::integral_constant<int, 2>{});
                } else {
                    // s += W2[:, j] h (+ the bias row of this tile: b2 on the first pair, zeros after it)
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) {
                        f32x4 acc[TW];
#pragma unroll
                        for (int tw = 0; tw < TW; ++tw) acc[tw] = xs[ft][tw];
                        if (has_bias && l == 1) {
                            const f32x4 bias = *reinterpret_cast<const f32x4*>(bl + 16 * ft);
#pragma unroll
                            for (int tw = 0; tw < TW; ++tw) acc[tw] += bias;
                        }
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            const u32x4 wa = *reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[ks]);
#pragma unroll
                            for (int tw = 0; tw < TW; ++tw) acc[tw] = M_::mma(wa, hb[ks][tw], acc[tw]);
                        }
#pragma unroll
                        for (int tw = 0; tw < TW; ++tw) xs[ft][tw] = acc[tw];
                    }
                }
                if (!resident) {
                    put(slot ^ 1);
                    __syncthreads();
                }
            }
        } else
        for (int l = 0; l < a.L; ++l, ++lcount) {
            const int slot = resident ? l : (lcount & 1);
            // ring: fetch the weights of the layer after this one (layer 0 of the next pass after the last)
            if (!resident) fetch(l + 1 < a.L ? l + 1 : 0);

            // B operands: the stream, packed
            u32x4 xb[KS][TW];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int tw = 0; tw < TW; ++tw) {
                    const f32x4 lo = xs[2 * ks][tw], hi = xs[2 * ks + 1][tw];
                    xb[ks][tw] = u32x4{M_::pack2(lo[0], lo[1]), M_::pack2(lo[2], lo[3]),
                                       M_::pack2(hi[0], hi[1]), M_::pack2(hi[2], hi[3])};
                }

            const bool act = (a.act_mask >> l) & 1u, add = (a.add_mask >> l) & 1u;
            const uint8_t* wb = smem + slot * WBUF + c16 * RS;
            // One layer for the wave's tokens.  ACT: 0 none, 1 tanh-GELU, 2 SiLU; ADD: the result is added to
            // the stream.  Both are compile-time here (the caller branches once per layer, uniformly), so the
            // epilogue has no selects and the last multiply of the activation fuses with the residual add.
            auto layer = [&](auto act_c, auto add_c) {
                constexpr int ACT = decltype(act_c)::value;
                constexpr bool ADD = decltype(add_c)::value;
                // the bias of a feature tile is requested two tiles ahead: it initialises the accumulators, so a load
                // issued where it is used would put a trip to the cache in front of every tile's first product
                const float* bl = bias0 + (size_t)l * C + 4 * g;
                f32x4 bias_q[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) bias_q[i] = vec4(bl + 16 * (i < FT ? i : 0), has_bias);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    const f32x4 bias = bias_q[ft & 1];
                    if (ft + 2 < FT) bias_q[ft & 1] = vec4(bl + 16 * (ft + 2), has_bias);
                    // The weight operands of a feature tile (one LDS read per k-step) are requested together at the head of
                    // the tile: left to itself the compiler, short of registers, issues each read where it is used, and
                    // every pair of products then starts with a round trip to LDS.  The fence keeps LDS reads from sinking
                    // below it and lets everything else cross (the epilogue of the tile before runs under this tile's
                    // reads).  Measured on the chain and the narrow-input modes; the expanding mode above is no faster for it.
                    u32x4 wq[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) wq[ks] = *reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[ks]);
                    __builtin_amdgcn_sched_barrier(0x7F);
                    f32x4 acc[TW];
#pragma unroll
                    for (int tw = 0; tw < TW; ++tw) acc[tw] = bias;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                        for (int tw = 0; tw < TW; ++tw) acc[tw] = M_::mma(wq[ks], xb[ks][tw], acc[tw]);
                    }
                    // tile ft of the stream is not an input of this layer any more once xb is packed
#pragma unroll
                    for (int tw = 0; tw < TW; ++tw) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float t = acc[tw][r];
                            if constexpr (ACT == 0) {
                                xs[ft][tw][r] = ADD ? xs[ft][tw][r] + t : t;
                            } else {
                                const float gate = ACT == 1 ? gelu_gate(t) : silu_gate(t);     // act(t) = t * gate
                                xs[ft][tw][r] = ADD ? fmaf(t, gate, xs[ft][tw][r]) : t * gate;
                            }
                        }
                    }
                }
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            if (!act) {
                if (add) layer(I0{}, std::true_type{}); else layer(I0{}, std::false_type{});
            } else if (a.act == 0) {
                if (add) layer(I1{}, std::true_type{}); else layer(I1{}, std::false_type{});
            } else {
                if (add) layer(I2{}, std::true_type{}); else layer(I2{}, std::false_type{});
            }
            if (!resident) {
                put(slot ^ 1);      // nobody reads that slot during this layer
                __syncthreads();
            }
        }

#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
            if (!live[tw]) continue;
            if (MODE == 2 && a.out_dim > 0) {
                // projecting last layer: only its first out_dim <= 4 rows are real, lane g == 0 holds them
                if (g == 0)
                    for (int r = 0; r < a.out_dim; ++r) {
                        const int64_t e = tok[tw] * a.ys + r;
                        const float o = xs[0][tw][r];
                        if (a.y_dtype == 0) static_cast<float*>(a.y)[e] = o;
                        else if (a.y_dtype == 1) static_cast<uint16_t*>(a.y)[e] = (uint16_t)Mm<bf16_t>::pack2(o, 0.f);
                        else static_cast<_Float16*>(a.y)[e] = (_Float16)o;
                    }
                continue;
            }
            if (MODE == 3 && a.y_head > 0) {
                // head-padded rows (columns as for x above): each head's channels, then zeros up to 16 columns,
                // written by the lane that holds the head's last four channels
                const int cf = a.y_head == 8 ? 32 : 64, c0 = a.y_head == 8 ? 8 * g - 4 * (g & 1) : 16 * g;
                const int nz = a.y_head == 8 ? ((g & 1) ? 2 : 0) : 3;        // groups of 4 zero columns behind this lane's channels
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                if (a.res) {
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) xs[ft][tw] += load4(a.res, tok[tw] * a.rs + 16 * ft + 4 * g, a.res_dtype);
                }
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    const int64_t col = tok[tw] * a.ys + ft * cf + c0;
                    store4(a.y, col, a.y_dtype, xs[ft][tw]);
                    for (int z = 1; z <= nz; ++z) store4(a.y, col + 4 * z, a.y_dtype, zero);
                }
                continue;
            }
            // all residual loads of the row before its first store: y may be the memory res points at, so a load
            // written after a store also stays behind it, and the row would take one trip to memory per tile
            if (a.res) {
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) xs[ft][tw] += load4(a.res, tok[tw] * a.rs + 16 * ft + 4 * g, a.res_dtype);
            }
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) store4(a.y, tok[tw] * a.ys + 16 * ft + 4 * g, a.y_dtype, xs[ft][tw]);
        }
    }
}

constexpr size_t kMlpLdsMax = 160 * 1024;   // all of a CU's LDS: five layers of 128 channels stay resident

template <typename T, int C, int TW, int WAVES, int MODE>
hipError_t launch_cte(const MlpArgs& a, hipStream_t st)
{
    auto kern = mlp_mfma_kernel<T, C, TW, WAVES, MODE>;
    const size_t wbuf = (size_t)C * C * 2;
    int resident = (size_t)a.L * wbuf <= kMlpLdsMax ? 1 : 0;
    size_t lds = (resident ? (size_t)a.L : 2) * wbuf;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess && resident) {      // the device grants less LDS than the layers need: stream them instead
        (void)hipGetLastError();
        resident = 0;
        lds = 2 * wbuf;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    }
    if (e != hipSuccess) return e;
    const int slots = resident_slots(reinterpret_cast<const void*>(kern), lds, 64 * WAVES);
    const int64_t per = 16 * TW * WAVES;
    const int64_t nblk = ((int64_t)a.T + per - 1) / per;
    const unsigned grid = (unsigned)(nblk < slots ? nblk : slots);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WAVES), lds, st, a, resident);
    return hipGetLastError();
}

template <typename T, int C, int TW, int WAVES>
hipError_t launch_ct(const MlpArgs& a, hipStream_t st)
{
    if (a.expand) return launch_cte<T, C, TW, WAVES, 1>(a, st);
    if (a.in_dim > 0 || a.out_dim > 0) return launch_cte<T, C, TW, WAVES, 2>(a, st);
    if (a.x_head > 0 || a.y_head > 0) return launch_cte<T, C, TW, WAVES, 3>(a, st);
    return launch_cte<T, C, TW, WAVES, 0>(a, st);
}

template <typename T>
hipError_t launch_t(const MlpArgs& a, hipStream_t st)
{
    // Few tokens: workgroups of 16 tokens per wave instead of 64 (32 at C = 128), four times as many of them.
    // Each one then re-reads its weight operands from LDS for every product, which costs throughput that a
    // launch too small to fill the chip does not need, and the layers' latency chain gets 4x (2x) shorter.
    const bool few = a.T < 32768;
    switch (a.C) {
        case 32:  return few ? launch_ct<T, 32, 1, 4>(a, st) : launch_ct<T, 32, 4, 4>(a, st);
        case 64:  return few ? launch_ct<T, 64, 1, 4>(a, st) : launch_ct<T, 64, 2, 4>(a, st);
        case 128: return few ? launch_ct<T, 128, 1, 8>(a, st) : launch_ct<T, 128, 2, 8>(a, st);
        default:  return hipErrorInvalidValue;
    }
}

}  // namespace

bool mlp_mfma_supported(int w_dtype, int C) { return (w_dtype == 1 || w_dtype == 2) && (C == 32 || C == 64 || C == 128); }

hipError_t launch_mlp_mfma(const MlpArgs& a, int w_dtype, hipStream_t st)
{
    return w_dtype == 1 ? launch_t<bf16_t>(a, st) : launch_t<f16_t>(a, st);
}

}  // namespace flare
