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

// Four stream values of a lane as separate registers.  As a 4-vector every single-element update copies the
// other three (the vector is one value to the compiler, and one register tuple), which the activation of a tile,
// element by element, would pay for with three moves per element.
struct Row4 {
    float e[4];
    __device__ __forceinline__ float& operator[](int i) { return e[i]; }
    __device__ __forceinline__ float operator[](int i) const { return e[i]; }
    __device__ __forceinline__ Row4& operator=(f32x4 v)
    {
        e[0] = v[0]; e[1] = v[1]; e[2] = v[2]; e[3] = v[3];
        return *this;
    }
    __device__ __forceinline__ Row4& operator+=(f32x4 v)
    {
        e[0] += v[0]; e[1] += v[1]; e[2] += v[2]; e[3] += v[3];
        return *this;
    }
    __device__ __forceinline__ operator f32x4() const { return f32x4{e[0], e[1], e[2], e[3]}; }
};

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

// Element type of a row (0 f32, 1 bf16, 2 f16) as a compile-time constant of the code that moves the row: the type is
// a launch argument, and a branch on it around every single load would put each load into a basic block of its own,
// where the 16-bit ones are followed by a wait for the data they convert -- one trip to memory per tile of a row.
// with_dtype branches once (uniformly) and runs a body in which all loads of a pass are issued back to back.
template <int DT> using Dt = std::integral_constant<int, DT>;
template <typename F> __device__ __forceinline__ void with_dtype(int dt, F&& f)
{
    if (dt == 0) f(Dt<0>{});
    else if (dt == 1) f(Dt<1>{});
    else f(Dt<2>{});
}

// four consecutive elements of a row as they lie in memory, and as fp32
template <int DT> struct Raw4 { using type = uint2; };
template <> struct Raw4<0> { using type = f32x4; };
template <int DT> __device__ __forceinline__ typename Raw4<DT>::type load4_raw(const void* base, int64_t elem)
{
    if constexpr (DT == 0) return *reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem);
    else return *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + elem);
}
template <int DT> __device__ __forceinline__ f32x4 unpack4(typename Raw4<DT>::type r)
{
    if constexpr (DT == 0) {
        return r;
    } else if constexpr (DT == 1) {
        return f32x4{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                     __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u)};
    } else {
        const f16x2 lo = __builtin_bit_cast(f16x2, r.x), hi = __builtin_bit_cast(f16x2, r.y);
        return f32x4{(float)lo[0], (float)lo[1], (float)hi[0], (float)hi[1]};
    }
}

template <int DT> __device__ __forceinline__ void store4(void* base, int64_t elem, f32x4 v)
{
    if constexpr (DT == 0) {
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + elem) = v;
    } else if constexpr (DT == 1) {
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
// 3 the chain with head-padded rows on either end.
// PF: 1 = the bias vectors of all layers stay in registers for the whole launch, element e in lane e % 64 of register
// e / 64, and reach the lanes that need them by ds_bpermute, which moves data through the LDS crossbar without touching
// LDS memory (all 160 KB hold weights).  No instruction of a layer then waits on the vector-memory counter, which retires
// in order: a bias load inside a layer waits for every older request, the row loads of the pass and the stores of the
// pass before included.  Resident weights only, PF_MAXL layers at most.
constexpr size_t kMlpLdsMax = 160 * 1024;   // all of a CU's LDS: five layers of 128 channels stay resident

template <int C> constexpr int pf_max_layers() { return 160 * 1024 / (C * C * 2) < 8 ? 160 * 1024 / (C * C * 2) : 8; }

template <typename T, int C, int TW, int WAVES, int MODE, int PF>
__global__ __launch_bounds__(64 * WAVES, (512 / (64 * WAVES) > 0 ? 512 / (64 * WAVES) : 1)) void mlp_mfma_kernel(MlpArgs a, int resident)
{
    static_assert(PF == 0 || MODE != 1, "the expanding mode streams its tiles through a ring");
    if constexpr (PF != 0) resident = 1;
    constexpr int PF_MAXL = pf_max_layers<C>();
    constexpr int NV = (C + 63) / 64;   // registers per parameter vector
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

    // PF: parameter vectors in registers; vec_at(v, ft) = elements 16 ft + 4 g .. + 3 of the vector
    uint32_t bv[PF ? PF_MAXL : 1][NV];
    if constexpr (PF != 0) {
        auto elem = [&](const float* p, bool have, int j) {
            const int e = 64 * j + lane;
            const float v = p[e < C ? e : 0];
            return have ? __float_as_uint(v) : 0u;
        };
#pragma unroll
        for (int l = 0; l < PF_MAXL; ++l)
#pragma unroll
            for (int j = 0; j < NV; ++j) bv[l][j] = elem(bias0 + (size_t)(l < a.L ? l : 0) * C, has_bias, j);
    }
    // The layer number is a run-time value and registers cannot be indexed by one (an indexed array would be placed in
    // scratch memory, whose loads count on the vector-memory counter as well): the bias vectors form a ring that
    // turns by one position per layer, so that the current layer's vector is always bv[0].
    auto rotate_bias = [&]() {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const uint32_t first = bv[0][j];
#pragma unroll
            for (int i = 0; i + 1 < (PF ? PF_MAXL : 1); ++i) bv[i][j] = bv[i + 1][j];
            bv[(PF ? PF_MAXL : 1) - 1][j] = first;
        }
    };
    int perm0 = 16 * g;     // byte address of lane 4 g in ds_bpermute's terms
    auto vec_at = [&](const uint32_t (&v)[NV], int ft) {
        const uint32_t src = v[(16 * ft) >> 6];
        f32x4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            o[r] = __int_as_float(__builtin_amdgcn_ds_bpermute(perm0 + 4 * ((16 * ft) & 63) + 4 * r, (int)src));
        return o;
    };

    int woff[KS];     // byte offset of this lane's chunk of k-step ks inside its weight row (swizzled)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) woff[ks] = ((4 * ks + g) ^ (c16 >> SWS)) << 4;
    // the same as LDS byte addresses of this lane's chunk in row c16 of slot 0 (the chain reads through these)
    uint32_t wa[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) wa[ks] = (uint32_t)(uintptr_t)smem + c16 * RS + woff[ks];

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

        // All loads of a pass's rows (both token tiles, every feature tile) are issued before the first is unpacked.
        // Rows of absent tokens are the last row's (tok is clamped), so nothing here depends on `live`.
        auto load_rows = [&](const void* base, int dt, int64_t stride, int cf, int c0, auto&& sink) {
            with_dtype(dt, [&](auto dc) {
                constexpr int DT = decltype(dc)::value;
                typename Raw4<DT>::type raw[FT][TW];
#pragma unroll
                for (int tw = 0; tw < TW; ++tw)
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) raw[ft][tw] = load4_raw<DT>(base, tok[tw] * stride + ft * cf + c0);
#pragma unroll
                for (int tw = 0; tw < TW; ++tw)
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) sink(ft, tw, unpack4<DT>(raw[ft][tw]));
            });
        };

        // the stream: lane (c16, g) holds features 16 ft + 4 g + r of token c16 of each tile
        Row4 xs[FT][TW];
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
            load_rows(a.x, a.x_dtype, a.xs, cf, c0, [&](int ft, int tw, f32x4 v) { xs[ft][tw] = v; });
        } else {
            load_rows(a.x, a.x_dtype, a.xs, 16, 4 * g, [&](int ft, int tw, f32x4 v) { xs[ft][tw] = v; });
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
            const uint32_t so = slot * WBUF;
            // One layer for the wave's tokens.  ACT: 0 none, 1 tanh-GELU, 2 SiLU; ADD: the result is added to
            // the stream.  Both are compile-time here (the caller branches once per layer, uniformly), so the
            // epilogue has no selects and the last multiply of the activation fuses with the residual add.
            auto layer = [&](auto act_c, auto add_c) {
                constexpr int ACT = decltype(act_c)::value;
                constexpr bool ADD = decltype(add_c)::value;
                // the bias of a feature tile is requested two tiles ahead: it initialises the accumulators, so a load
                // issued where it is used would put a trip to the cache in front of every tile's first product
                const float* bl = bias0 + (size_t)l * C + 4 * g;
                auto bias_at = [&](int ft) {
                    if constexpr (PF != 0) return vec_at(bv[0], ft);    // the ring of bias vectors has this layer's in front
                    else return vec4(bl + 16 * ft, has_bias);
                };
                // Software pipeline over the feature tiles, written out: step ft issues the products of tile ft in between
                // the activations of tile ft - 1, group by group, and requests the weight operands of tile ft + 1 (one
                // LDS read per k-step) and the bias of tile ft + 2 ahead, so that no product waits for LDS and no
                // activation for a product issued just before it.  The fences pin the interleaving (everything may move
                // inside a group, nothing across).  By itself this order measured the same as source order (reads, a
                // wait, the products, a wait, the activations): with two waves per SIMD each covers the other's waits.
                // What the chain gained (9 % at five layers of 128 channels) came from taking the bias loads out of the
                // layers (PF above); the written-out order is kept because it holds the registers of a tile to one set of
                // weight operands and two sets of accumulators, which is what lets the bias vectors stay resident.
                auto rd = [&](int ft, int ks) {
                    typedef const u32x4 __attribute__((address_space(3))) * lds_ptr;
                    return *(lds_ptr)(uintptr_t)(wa[ks] + so + (16 * ft) * RS);
                };
                constexpr int NP = KS * TW, NE = TW * 4;      // products and activations per tile
                constexpr int GS = 2;                           // per group: GS activations and their share of the products
                constexpr int NG = NE / GS;
                // one set of weight operands: the operand of k-step ks is requested for the next tile right behind the
                // last product that reads it for this one
                u32x4 wq[KS];
                f32x4 bias_q[2], accp[TW];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) wq[ks] = rd(0, ks);
#pragma unroll
                for (int i = 0; i < 2; ++i) bias_q[i] = bias_at(i < FT ? i : 0);
#pragma unroll
                for (int ft = 0; ft <= FT; ++ft) {
                    f32x4 acc[TW];
                    if (ft < FT) {
#pragma unroll
                        for (int tw = 0; tw < TW; ++tw) acc[tw] = bias_q[ft & 1];
                        if (ft + 2 < FT) bias_q[ft & 1] = bias_at(ft + 2);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi) {
                        if (ft < FT) {
#pragma unroll
                            for (int i = gi * NP / NG; i < (gi + 1) * NP / NG; ++i) {
                                const int ks = i / TW, tw = i % TW;
                                acc[tw] = M_::mma(wq[ks], xb[ks][tw], acc[tw]);
                                if (tw == TW - 1 && ft + 1 < FT) wq[ks] = rd(ft + 1, ks);
                            }
                        }
                        if (ft > 0) {
                            // tile ft - 1 of the stream is not an input of this layer any more once xb is packed
#pragma unroll
                            for (int i = gi * GS; i < (gi + 1) * GS; ++i) {
                                const int tw = i % TW, r = i / TW;
                                const float t = accp[tw][r];
                                const float o = xs[ft - 1][tw][r];
                                if constexpr (ACT == 0) {
                                    xs[ft - 1][tw][r] = ADD ? o + t : t;
                                } else {
                                    const float gate = ACT == 1 ? gelu_gate(t) : silu_gate(t);     // act(t) = t * gate
                                    xs[ft - 1][tw][r] = ADD ? fmaf(t, gate, o) : t * gate;
                                }
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int tw = 0; tw < TW; ++tw) accp[tw] = acc[tw];
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
            if constexpr (PF != 0) rotate_bias();
        }
        if constexpr (PF != 0)
            for (int l = a.L; l < PF_MAXL; ++l) rotate_bias();     // back to layer 0 in front for the next pass

        if (MODE == 2 && a.out_dim > 0) {
            // projecting last layer: only its first out_dim <= 4 rows are real, lane g == 0 holds them
#pragma unroll
            for (int tw = 0; tw < TW; ++tw) {
                if (!live[tw] || g != 0) continue;
#pragma unroll
                for (int r = 0; r < 4; ++r) {       // r is a constant of each copy: a run-time index would move the stream to scratch
                    if (r >= a.out_dim) continue;
                    const int64_t e = tok[tw] * a.ys + r;
                    const float o = xs[0][tw][r];
                    if (a.y_dtype == 0) static_cast<float*>(a.y)[e] = o;
                    else if (a.y_dtype == 1) static_cast<uint16_t*>(a.y)[e] = (uint16_t)Mm<bf16_t>::pack2(o, 0.f);
                    else static_cast<_Float16*>(a.y)[e] = (_Float16)o;
                }
            }
            continue;
        }
        // all residual loads of a pass before its first store: y may be the memory res points at, so a load written
        // after a store also stays behind it, and the rows would take one trip to memory per tile
        if (a.res) load_rows(a.res, a.res_dtype, a.rs, 16, 4 * g, [&](int ft, int tw, f32x4 v) { xs[ft][tw] += v; });
        with_dtype(a.y_dtype, [&](auto dc) {
            constexpr int DT = decltype(dc)::value;
            if (MODE == 3 && a.y_head > 0) {
                // head-padded rows (columns as for x above): each head's channels, then zeros up to 16 columns,
                // written by the lane that holds the head's last four channels
                const int cf = a.y_head == 8 ? 32 : 64, c0 = a.y_head == 8 ? 8 * g - 4 * (g & 1) : 16 * g;
                const int nz = a.y_head == 8 ? ((g & 1) ? 2 : 0) : 3;        // groups of 4 zero columns behind this lane's channels
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int tw = 0; tw < TW; ++tw) {
                    if (!live[tw]) continue;
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) {
                        const int64_t col = tok[tw] * a.ys + ft * cf + c0;
                        store4<DT>(a.y, col, xs[ft][tw]);
                        for (int z = 1; z <= nz; ++z) store4<DT>(a.y, col + 4 * z, zero);
                    }
                }
            } else {
#pragma unroll
                for (int tw = 0; tw < TW; ++tw) {
                    if (!live[tw]) continue;
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) store4<DT>(a.y, tok[tw] * a.ys + 16 * ft + 4 * g, xs[ft][tw]);
                }
            }
        });
    }
}


template <typename T, int C, int TW, int WAVES, int MODE, int PF>
hipError_t launch_pf(const MlpArgs& a, hipStream_t st)
{
    auto kern = mlp_mfma_kernel<T, C, TW, WAVES, MODE, PF>;
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
    if (PF != 0 && !resident) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WAVES), lds, st, a, resident);
    return hipGetLastError();
}

// Picks the instance with the bias vectors in registers where it applies: many tokens per workgroup (TW > 1 marks
// those launches) and weights that stay resident.
template <typename T, int C, int TW, int WAVES, int MODE>
hipError_t launch_cte(const MlpArgs& a, hipStream_t st)
{
    if constexpr (MODE != 1 && TW > 1) {
        if ((size_t)a.L * C * C * 2 <= kMlpLdsMax && a.L <= pf_max_layers<C>()) {
            const hipError_t e = launch_pf<T, C, TW, WAVES, MODE, 1>(a, st);
            if (e != hipErrorInvalidValue) return e;
            (void)hipGetLastError();
        }
    }
    return launch_pf<T, C, TW, WAVES, MODE, 0>(a, st);
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
    // Up to 32,768 tokens inclusive: at C = 128 that is one workgroup of 128 tokens on each of 256 CUs, where the
    // many-token instance would occupy half of them (five layers: 20.6 against 24.0 us; at 49,152 tokens 32.9 against 24.8).
    const bool few = a.T <= 32768;
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
