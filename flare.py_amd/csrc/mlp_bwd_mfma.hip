// Backward of the fused token-wise MLP stack of mlp_mfma.hip (the chain of C x C layers; bf16 / f16 weights,
// C in {32, 64, 128}): what torch autograd does for  y = res + ResidualMLP(norm(x))  of
// pdebench/models/flare.py:45-59 and 204-215, in one token-parallel launch plus reductions over tokens for the parameters.
//
// Forward, per token:  s_0 = norm(x);  layer l:  t_l = W_l s_l + b_l,  u_l = act(t_l) if bit l of act_mask else t_l,
// s_{l+1} = s_l + u_l if bit l of add_mask else u_l;  y = res + s_L.
// Backward, given dy:  ds_L = dy;  for l = L-1 .. 0:  dt_l = ds_{l+1} * act'(t_l),
// ds_l = (ds_{l+1} if add) + W_l^T dt_l;  then the norm's backward gives dx.  Parameter gradients:
//   dW_l = sum_t dt_l s_l^T,   db_l = sum_t dt_l,   dgamma = sum_t ds_0 * xhat,   dbeta = sum_t ds_0.
//
// The kernel recomputes the forward for its 16-token tile (same layout as mlp_mfma.hip: the product is taken
// transposed, lane = token, the accumulators of one layer packed to 16 bits are the B operands of the next), keeps
// act'(t_l) of every layer packed to 16 bits in registers, and walks the chain back with the TRANSPOSED weights in
// the place of the weights (ds_l^T = W_l^T dt_l^T is the same product shape).  What a reduction over all tokens
// needs leaves the kernel as 16-bit rows: s_l (the input of every layer) and dt_l, from which the caller forms
// dW_l = dt_l^T s_l and db_l are formed in one pass by mlp_wgrad_mfma.hip; for the norm's parameters the kernel
// leaves ds_0 as 16-bit rows and every token's (mean, 1/std), and mlp_norm_grads_kernel sums dgamma, dbeta over token
// ranges into one partial row per workgroup (summed in a fixed order by a last small launch: no atomics).
// Weights move through LDS: all 2 L tiles resident when they fit, else a two-slot ring in the order
// W_0 .. W_{L-1}, W_{L-1}^T .. W_0^T with one barrier per layer; they arrive as LDS images and are loaded straight
// into their slots.
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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mw;
template <> struct Mw<bf16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float lo(uint32_t p) { return __uint_as_float(p << 16); }
    static __device__ __forceinline__ float hi(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }
};
template <> struct Mw<f16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float lo(uint32_t p) { return (float)__builtin_bit_cast(f16x2, p)[0]; }
    static __device__ __forceinline__ float hi(uint32_t p) { return (float)__builtin_bit_cast(f16x2, p)[1]; }
};

// Element type of a row (0 f32, 1 bf16, 2 f16) as a compile-time constant of the code that moves the row: the type is
// a launch argument, and a branch on it around every single load puts each load into a basic block of its own, where a
// wait for everything in flight precedes the next -- one trip to memory per feature tile of a row instead of one per
// row.  with_dtype branches once (uniformly); load_row issues all loads of a row back to back and unpacks afterwards.
template <typename F> __device__ __forceinline__ void with_dtype(int dt, F&& f)
{
    if (dt == 0) f(std::integral_constant<int, 0>{});
    else if (dt == 1) f(std::integral_constant<int, 1>{});
    else f(std::integral_constant<int, 2>{});
}
template <int DT> struct Raw4 { using type = uint2; };
template <> struct Raw4<0> { using type = f32x4; };
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
// tiles ft = 0 .. FT-1 of a row: four elements each, 16 apart, from element elem0 on; sink(ft, values)
template <int FT, typename F>
__device__ __forceinline__ void load_row(const void* base, int dt, int64_t elem0, F&& sink)
{
    with_dtype(dt, [&](auto dc) {
        constexpr int DT = decltype(dc)::value;
        typename Raw4<DT>::type raw[FT];
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) {
            if constexpr (DT == 0) raw[ft] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem0 + 16 * ft);
            else raw[ft] = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + elem0 + 16 * ft);
        }
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) sink(ft, unpack4<DT>(raw[ft]));
    });
}

__device__ __forceinline__ void st4(void* base, int64_t elem, int dt, f32x4 v)
{
    if (dt == 0) {
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + elem) = v;
    } else if (dt == 1) {
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + elem) =
            make_uint2(Mw<bf16_t>::pack2(v[0], v[1]), Mw<bf16_t>::pack2(v[2], v[3]));
    } else {
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + elem) =
            make_uint2(Mw<f16_t>::pack2(v[0], v[1]), Mw<f16_t>::pack2(v[2], v[3]));
    }
}

__device__ __forceinline__ float tok_sum(float v)   // sum over the 4 lane groups that share a token
{
    v = sum_xor16(v);
    v = sum_xor32(v);
    return v;
}

// A packed operand quad {lo01, lo23, hi01, hi23} holds channels 4g..4g+3 of two feature tiles 16 channels apart.
// Lanes 16 apart (g and g ^ 1) exchange halves, after which every lane holds eight consecutive channels: those
// starting at row_col(g) = 0, 16, 8, 24 for g = 0..3.  A token's row then leaves as 16-byte pieces, 64 contiguous
// bytes per store instruction, instead of 8-byte pieces that cover 32.  All lanes of the wave must be active.
__device__ __forceinline__ u32x4 row_piece(u32x4 q)
{
    const auto r0 = __builtin_amdgcn_permlane16_swap(q[0], q[2], false, false);
    const auto r1 = __builtin_amdgcn_permlane16_swap(q[1], q[3], false, false);
    return u32x4{r0[0], r1[0], r0[1], r1[1]};
}
__device__ __forceinline__ int row_col(int g) { return (g & 1) ? 12 + 4 * g : 4 * g; }

// A [T,C] 16-bit row array receives a wave's 16 tokens from packed operand quads.  After row_piece a token's four
// lanes hold 64 contiguous bytes per k-step; the two half-rows of 8 lanes then trade pieces of neighbouring k-steps
// (one rotate by 8 within each 16 lanes), so that one store instruction completes 128-byte lines: the first for
// tokens 0-7 of the tile, the second for tokens 8-15.  t: the lane's token, n_tok: tokens in the array.  All lanes
// of the wave must be active.
template <int C>
__device__ __forceinline__ void store_rows(uint16_t* base, const u32x4* q, int64_t t, int64_t n_tok, int g, int c16)
{
    constexpr int KS = C / 32;
    u32x4 piece[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) piece[ks] = row_piece(q[ks]);
    const int rc = row_col(g);
    if constexpr (KS == 1) {
        if (t < n_tok) *reinterpret_cast<u32x4*>(base + (size_t)t * C + rc) = piece[0];
    } else {
        const bool low = c16 < 8;
#pragma unroll
        for (int kp = 0; kp < KS; kp += 2) {
            u32x4 send, recv, va, vb;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                send[r] = low ? piece[kp + 1][r] : piece[kp][r];
                recv[r] = __builtin_amdgcn_update_dpp(send[r], send[r], 0x128, 0xf, 0xf, false);     // row_ror:8
                va[r] = low ? piece[kp][r] : recv[r];
                vb[r] = low ? recv[r] : piece[kp + 1][r];
            }
            const int64_t ta = low ? t : t - 8, tb = low ? t + 8 : t;
            const int col = 32 * (low ? kp : kp + 1) + rc;
            if (ta < n_tok) *reinterpret_cast<u32x4*>(base + (size_t)ta * C + col) = va;
            if (tb < n_tok) *reinterpret_cast<u32x4*>(base + (size_t)tb * C + col) = vb;
        }
    }
}

// act(t) = t * gate and its derivative.  tanh-GELU: gate = sigmoid(2u), 2u = t (1.5957691 + 0.0713548 t^2), so
// act' = gate (1 + t (1 - gate) (1.5957691 + 0.2140645 t^2));  SiLU: gate = sigmoid(t), act' = gate (1 + t (1 - gate)).
template <int ACT>
__device__ __forceinline__ void act_and_slope(float t, float& value, float& slope)
{
    if (ACT == 1) {
        const float t2 = t * t;
        const float gate = __builtin_amdgcn_rcpf(1.f + fast_exp2(-t * (2.3022081f + 0.10294324f * t2)));
        value = t * gate;
        slope = gate * fmaf(t * (1.f - gate), fmaf(0.2140645f, t2, 1.5957691f), 1.f);
    } else {
        const float gate = __builtin_amdgcn_rcpf(1.f + fast_exp2(-kLog2e * t));
        value = t * gate;
        slope = gate * fmaf(t, 1.f - gate, 1.f);
    }
}

// LMAX: the layers are unrolled up to this count (their saved slopes live in registers), a.L <= LMAX.
template <typename T, int C, int WAVES, int LMAX>
__global__ __launch_bounds__(64 * WAVES, 1) void mlp_bwd_kernel(MlpBwdArgs a, int resident)
{
    constexpr int NT = 64 * WAVES;
    constexpr int NCH = (C * C / 8 + NT - 1) / NT;   // 16-byte weight chunks per thread and tile
    constexpr int FT = C / 16;        // feature tiles of the stream
    constexpr int KS = C / 32;        // k-steps of one layer
    constexpr int RS = C * 2;         // LDS row stride in bytes (16-byte chunks XOR-swizzled with the row number)
    constexpr int WBUF = C * RS;
    constexpr int CPR = C / 8;
    constexpr int SWS = CPR == 16 ? 0 : CPR == 8 ? 1 : 2;
    using M_ = Mw<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    // bias rows of every layer, then gamma and beta, as fp32 in LDS: read from there the values cost no vector-memory
    // slot (a global load in the middle of a step would queue behind the weight tile requested at its start)
    __shared__ __attribute__((aligned(16))) float pvec[(LMAX + 2) * C];

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);       // the wave number, known to be uniform
    const int L = a.L;
    for (int i = tid; i < (LMAX + 2) * C; i += NT) {
        const int row = i / C, c = i % C;
        float v = 0.f;
        if (row < LMAX) { if (a.bias && row < L) v = a.bias[(size_t)row * C + c]; }
        else if (row == LMAX) { if (a.norm != 0) v = a.gamma[c]; }
        else if (a.norm != 0 && a.beta) v = a.beta[c];
        pvec[i] = v;
    }

    // Weight tile of ring step q: W_q for q < L (forward), W_{2L-1-q}^T after that (backward).  The caller hands
    // the tiles over as LDS images (the 16-bit elements already in the order the A-operand reads expect, see
    // mlp_weight_image in the host code), so a tile goes from global memory straight into its slot, 16 bytes per
    // lane, with no registers and no LDS stores in between.
    auto stage = [&](int q, int slot) {
        const uint8_t* img = reinterpret_cast<const uint8_t*>(q < L ? a.w + (size_t)q * C * C : a.wt + (size_t)(2 * L - 1 - q) * C * C);
        // The lane's byte offset passes through an empty asm statement so that the 64-bit address of each (tile,
        // chunk) is formed here, with one add, and not ahead of the token loop: kept across the loop those addresses
        // would be 8 * L * NCH registers that end up in scratch memory, and each reload from there waits for every
        // vector-memory operation in flight, the previous chunk's load included.
        uint32_t loff = lane * 16;
        asm volatile("" : "+v"(loff));
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c0 = i * NT + w * 64;           // first 16-byte chunk of this wave's share (uniform over the wave)
            if ((C * C / 8) % NT == 0 || c0 < C * C / 8)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(img + (size_t)c0 * 16 + loff),
                                                 (__attribute__((address_space(3))) void*)(smem + slot * WBUF + c0 * 16), 16, 0, 0);
        }
    };
    auto staged = [&]() {       // the workgroup's loads have landed and are visible to all its waves
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };
    int woff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) woff[ks] = ((4 * ks + g) ^ (c16 >> SWS)) << 4;

    int qcount = 0;      // ring mode: steps done by this workgroup; its parity names the slot in use
    if (resident) {
        for (int q = 0; q < 2 * L; ++q) stage(q, q);
    } else {
        stage(0, 0);
    }
    staged();

    // one product of a layer: out tile ft = init + (weight tile of the current ring slot) x (packed operand)
    auto ring_step_begin = [&](int q) -> const uint8_t* {
        const int slot = resident ? q : (qcount & 1);
        // ring: the next step's tile goes into the other slot, which nobody has read since the last barrier
        if (!resident) stage(q + 1 < 2 * L ? q + 1 : 0, slot ^ 1);
        return smem + slot * WBUF + c16 * RS;
    };
    auto ring_step_end = [&]() {
        if (!resident) staged();
        ++qcount;
    };

    // The waves of a workgroup move in step (one barrier per layer), so a trip to memory that one of them waits for
    // is a trip all of them wait for.  The rows of x are therefore requested where registers are free and nothing
    // waits for them yet: the next tile's row while this tile's norm is walked back (x_next), and this tile's row
    // again, for that walk, at the start of the last backward step (x_again), when the slopes of the later layers
    // are dead.
    const int64_t nblk = ((int64_t)a.T + WAVES * 16 - 1) / (WAVES * 16);
    auto row_of = [&](int64_t blk) {
        const int64_t t = blk * (WAVES * 16) + w * 16 + c16;
        return t < a.T ? t : a.T - 1;
    };
    f32x4 x_next[FT];
    {
        const int64_t r = row_of(blockIdx.x);           // blockIdx.x < nblk: the grid is never larger
        load_row<FT>(a.x, a.x_dtype, r * a.xs + 4 * g, [&](int ft, f32x4 v) { x_next[ft] = v; });
    }
    for (int64_t blk = blockIdx.x; blk < nblk; blk += gridDim.x) {
        const int64_t t = blk * (WAVES * 16) + w * 16 + c16;
        const bool live = t < a.T;
        const int64_t tok = live ? t : a.T - 1;

        // ---- forward, recomputed: the stream, the inputs of every layer, the slopes of every activation ----
        f32x4 xs[FT];
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) xs[ft] = x_next[ft];
        float mean = 0.f, rstd = 1.f;
        if (a.norm != 0) {
            float s = 0.f;
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) s += xs[ft][0] + xs[ft][1] + xs[ft][2] + xs[ft][3];
            const float rowmean = tok_sum(s) * (1.f / C);
            mean = a.norm == 1 ? rowmean : 0.f;
            float ss = 0.f;
#pragma unroll
            for (int ft = 0; ft < FT; ++ft)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float d = xs[ft][r] - mean;
                    ss = fmaf(d, d, ss);
                }
            rstd = rsqrtf(tok_sum(ss) * (1.f / C) + a.eps);
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 gm = *reinterpret_cast<const f32x4*>(pvec + LMAX * C + 16 * ft + 4 * g);
                const f32x4 bt = *reinterpret_cast<const f32x4*>(pvec + (LMAX + 1) * C + 16 * ft + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) xs[ft][r] = (xs[ft][r] - mean) * rstd * gm[r] + bt[r];
            }
        }

        uint32_t slope[LMAX][FT][2];      // act'(t_l), packed to 16 bits (layers without activation: unused)
#pragma unroll
        for (int l = 0; l < LMAX; ++l) {
            if (l >= L) break;
            u32x4 xb[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const f32x4 lo = xs[2 * ks], hi = xs[2 * ks + 1];
                xb[ks] = u32x4{M_::pack2(lo[0], lo[1]), M_::pack2(lo[2], lo[3]), M_::pack2(hi[0], hi[1]), M_::pack2(hi[2], hi[3])};
            }
            store_rows<C>(a.a_in + (size_t)l * a.T * C, xb, t, a.T, g, c16);      // s_l, the input of layer l, as a 16-bit row (for dW_l)
            const uint8_t* wb = ring_step_begin(l);
            const bool act = (a.act_mask >> l) & 1u, add = (a.add_mask >> l) & 1u;
            auto layer = [&](auto act_c, auto add_c) {
                constexpr int ACT = decltype(act_c)::value;
                constexpr bool ADD = decltype(add_c)::value;
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    f32x4 acc = *reinterpret_cast<const f32x4*>(pvec + l * C + 16 * ft + 4 * g);
                    // the tile's weight operands requested together: read where they are used, every product starts with
                    // a round trip to LDS (the fence holds LDS reads in place and lets everything else cross)
                    u32x4 wq[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) wq[ks] = *reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[ks]);
                    __builtin_amdgcn_sched_barrier(0x7F);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) acc = M_::mma(wq[ks], xb[ks], acc);
                    float sl[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float u = acc[r];
                        sl[r] = 1.f;
                        if constexpr (ACT != 0) act_and_slope<ACT>(acc[r], u, sl[r]);
                        xs[ft][r] = ADD ? xs[ft][r] + u : u;
                    }
                    slope[l][ft][0] = M_::pack2(sl[0], sl[1]);
                    slope[l][ft][1] = M_::pack2(sl[2], sl[3]);
                    // two feature tiles at a time: without a fence the scheduler lifts the operand reads of all
                    // tiles to the front and the slopes of five layers no longer fit beside them
                    if (C == 128 && (ft & 1)) __builtin_amdgcn_sched_barrier(0);
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
            ring_step_end();
        }

        // ---- backward through the chain: xs becomes ds ----
        f32x4 x_again[FT];
        load_row<FT>(a.dy, a.dy_dtype, tok * a.dys + 4 * g, [&](int ft, f32x4 v) { xs[ft] = live ? v : f32x4{0.f, 0.f, 0.f, 0.f}; });
#pragma unroll
        for (int l = LMAX - 1; l >= 0; --l) {
            if (l >= L) continue;
            if (l == 0 && a.norm != 0) {
                load_row<FT>(a.x, a.x_dtype, tok * a.xs + 4 * g, [&](int ft, f32x4 v) { x_again[ft] = v; });
            }
            const uint8_t* wb = ring_step_begin(2 * L - 1 - l);
            const bool act = (a.act_mask >> l) & 1u, add = (a.add_mask >> l) & 1u;
            // dt_l = ds_{l+1} * act'(t_l), packed: the B operands of this product and the rows kept for dW_l, db_l
            u32x4 db[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x4 lo = xs[2 * ks], hi = xs[2 * ks + 1];
                if (act) {
                    const uint32_t* s0 = slope[l][2 * ks];
                    const uint32_t* s1 = slope[l][2 * ks + 1];
                    lo[0] *= M_::lo(s0[0]); lo[1] *= M_::hi(s0[0]); lo[2] *= M_::lo(s0[1]); lo[3] *= M_::hi(s0[1]);
                    hi[0] *= M_::lo(s1[0]); hi[1] *= M_::hi(s1[0]); hi[2] *= M_::lo(s1[1]); hi[3] *= M_::hi(s1[1]);
                }
                db[ks] = u32x4{M_::pack2(lo[0], lo[1]), M_::pack2(lo[2], lo[3]), M_::pack2(hi[0], hi[1]), M_::pack2(hi[2], hi[3])};
            }
            store_rows<C>(a.g_out + (size_t)l * a.T * C, db, t, a.T, g, c16);
            // ds_l = (ds_{l+1} if the layer added to the stream) + W_l^T dt_l
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                f32x4 acc = add ? xs[ft] : f32x4{0.f, 0.f, 0.f, 0.f};
                u32x4 wq[KS];      // requested together, as above (two tiles at a time, their chains alternating, is no faster)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) wq[ks] = *reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[ks]);
                __builtin_amdgcn_sched_barrier(0x7F);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = M_::mma(wq[ks], db[ks], acc);
                xs[ft] = acc;
                if (C == 128 && (ft & 1)) __builtin_amdgcn_sched_barrier(0);
            }
            ring_step_end();
        }

        // ---- the norm's backward, dx ----
        {   // without a condition (the last tile reads its own row once more): under one, the registers of x_next
            // would have to keep their old value through the whole tile
            const int64_t r = row_of(blk + gridDim.x < nblk ? blk + gridDim.x : blk);
            load_row<FT>(a.x, a.x_dtype, r * a.xs + 4 * g, [&](int ft, f32x4 v) { x_next[ft] = v; });
        }
        if (a.norm != 0) {
            // ds_0 and the token's statistics go out for dgamma, dbeta; xhat is taken again from x (x_again) rather
            // than kept in registers through the chain;  g = ds_0 * gamma
            u32x4 dq[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const f32x4 lo = xs[2 * ks], hi = xs[2 * ks + 1];
                dq[ks] = u32x4{M_::pack2(lo[0], lo[1]), M_::pack2(lo[2], lo[3]), M_::pack2(hi[0], hi[1]), M_::pack2(hi[2], hi[3])};
            }
            store_rows<C>(a.dn, dq, t, a.T, g, c16);
            if (live && lane < 16) *reinterpret_cast<float2*>(a.stats + 2 * tok) = make_float2(mean, rstd);
            float m1 = 0.f, m2 = 0.f;
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 xr = x_again[ft];
                const f32x4 gm = *reinterpret_cast<const f32x4*>(pvec + LMAX * C + 16 * ft + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    xs[ft][r] *= gm[r];
                    m1 += xs[ft][r];
                    m2 = fmaf(xs[ft][r], (xr[r] - mean) * rstd, m2);
                }
            }
            m1 = a.norm == 1 ? tok_sum(m1) * (1.f / C) : 0.f;
            m2 = tok_sum(m2) * (1.f / C);
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 xr = x_again[ft];
#pragma unroll
                for (int r = 0; r < 4; ++r) xs[ft][r] = rstd * (xs[ft][r] - m1 - (xr[r] - mean) * rstd * m2);
            }
        }
        if (live) {
            // every load of dy before the first store of dx (a load written after a store stays behind it: the two
            // may be the same memory as far as the compiler knows)
            if (a.add_dy & 1) {
                load_row<FT>(a.dy, a.dy_dtype, tok * a.dys + 4 * g, [&](int ft, f32x4 v) { xs[ft] += v; });
            }
            if (a.add_dy & 2) {     // dx holds another path's gradient of the same x: the sum goes back
                load_row<FT>(a.dx, a.dx_dtype, tok * a.dxs + 4 * g, [&](int ft, f32x4 v) { xs[ft] += v; });
            }
            with_dtype(a.dx_dtype, [&](auto dc) {
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) st4(a.dx, tok * a.dxs + 16 * ft + 4 * g, decltype(dc)::value, xs[ft]);
            });
        }
    }
}

// Backward of the expanding two-layer MLP  y = res + W2 act(W1 norm(x) + b1) + b2  (the "4x" feed-forward block; the
// forward is mode 1 of mlp_mfma.hip, hidden width E * C run as E chunks of C).  Per chunk j and 16-token tile:
//   t_j = W1[j] n + b1[j],  h_j = act(t_j)                       (recomputed; tile 2 j of a.w)
//   dh_j = W2[:,j]^T dy,    dt_j = dh_j * act'(t_j)              (tile 2 j + 1 of a.wt)
//   dn  += W1[j]^T dt_j                                          (tile 2 j of a.wt)
// three ring steps per chunk, nothing kept from one chunk to the next but dn.  Rows left for the weight gradients:
// n and dy in 16 bits (one row array each, shared by all chunks), h_j (a.a_in) and dt_j (a.g_out) per chunk:
//   dW1[j] = dt_j^T n,  db1[j] = column sums of dt_j,  dW2[:,j] = dy^T h_j,  db2 = column sums of dy.
constexpr int kExpandMax = 8;
template <typename T, int C, int WAVES>
__global__ __launch_bounds__(64 * WAVES, 1) void mlp_bwd_expand_kernel(MlpBwdArgs a)
{
    constexpr int NT = 64 * WAVES;
    constexpr int NCH = (C * C / 8 + NT - 1) / NT;
    constexpr int FT = C / 16, KS = C / 32, RS = C * 2, WBUF = C * RS, CPR = C / 8;
    constexpr int SWS = CPR == 16 ? 0 : CPR == 8 ? 1 : 2;
    constexpr int PG = kExpandMax, PB = kExpandMax + 1;          // rows of pvec: b1[0..E), gamma, beta
    using M_ = Mw<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ __attribute__((aligned(16))) float pvec[(kExpandMax + 2) * C];

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int E = a.E, Q = 3 * E;
    for (int i = tid; i < (kExpandMax + 2) * C; i += NT) {
        const int row = i / C, c = i % C;
        float v = 0.f;
        if (row < kExpandMax) { if (a.bias && row < E) v = a.bias[(size_t)(2 * row) * C + c]; }
        else if (row == PG) { if (a.norm != 0) v = a.gamma[c]; }
        else if (a.norm != 0 && a.beta) v = a.beta[c];
        pvec[i] = v;
    }

    auto stage = [&](int q, int slot) {
        const int j = q / 3, r = q - 3 * j;
        const uint16_t* tile = r == 0 ? a.w + (size_t)(2 * j) * C * C : a.wt + (size_t)(2 * j + (r == 1 ? 1 : 0)) * C * C;
        const uint8_t* img = reinterpret_cast<const uint8_t*>(tile);
        uint32_t loff = lane * 16;
        asm volatile("" : "+v"(loff));      // the address of a chunk is formed here, not kept across the token loop
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c0 = i * NT + w * 64;
            if ((C * C / 8) % NT == 0 || c0 < C * C / 8)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(img + (size_t)c0 * 16 + loff),
                                                 (__attribute__((address_space(3))) void*)(smem + slot * WBUF + c0 * 16), 16, 0, 0);
        }
    };
    auto staged = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };
    int woff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) woff[ks] = ((4 * ks + g) ^ (c16 >> SWS)) << 4;

    auto pack4 = [](const f32x4& lo, const f32x4& hi) {
        return u32x4{M_::pack2(lo[0], lo[1]), M_::pack2(lo[2], lo[3]), M_::pack2(hi[0], hi[1]), M_::pack2(hi[2], hi[3])};
    };

    int qcount = 0;
    stage(0, 0);
    staged();
    auto step_begin = [&](int q) -> const uint8_t* {
        const int slot = qcount & 1;
        stage(q + 1 < Q ? q + 1 : 0, slot ^ 1);
        return smem + slot * WBUF + c16 * RS;
    };
    auto step_end = [&]() {
        staged();
        ++qcount;
    };

    const int64_t nblk = ((int64_t)a.T + WAVES * 16 - 1) / (WAVES * 16);
    for (int64_t blk = blockIdx.x; blk < nblk; blk += gridDim.x) {
        const int64_t t = blk * (WAVES * 16) + w * 16 + c16;
        const bool live = t < a.T;
        const int64_t tok = live ? t : a.T - 1;

        // n = norm(x) and dy, both packed once as B operands and left as 16-bit rows
        f32x4 xs[FT];
        load_row<FT>(a.x, a.x_dtype, tok * a.xs + 4 * g, [&](int ft, f32x4 v) { xs[ft] = v; });
        float mean = 0.f, rstd = 1.f;
        if (a.norm != 0) {
            float s = 0.f;
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) s += xs[ft][0] + xs[ft][1] + xs[ft][2] + xs[ft][3];
            const float rowmean = tok_sum(s) * (1.f / C);
            mean = a.norm == 1 ? rowmean : 0.f;
            float ss = 0.f;
#pragma unroll
            for (int ft = 0; ft < FT; ++ft)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float d = xs[ft][r] - mean;
                    ss = fmaf(d, d, ss);
                }
            rstd = rsqrtf(tok_sum(ss) * (1.f / C) + a.eps);
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 gm = *reinterpret_cast<const f32x4*>(pvec + PG * C + 16 * ft + 4 * g);
                const f32x4 bt = *reinterpret_cast<const f32x4*>(pvec + PB * C + 16 * ft + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) xs[ft][r] = (xs[ft][r] - mean) * rstd * gm[r] + bt[r];
            }
        }
        u32x4 nb[KS], dyb[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) nb[ks] = pack4(xs[2 * ks], xs[2 * ks + 1]);
        store_rows<C>(a.n_row, nb, t, a.T, g, c16);
        load_row<FT>(a.dy, a.dy_dtype, tok * a.dys + 4 * g, [&](int ft, f32x4 v) { xs[ft] = live ? v : f32x4{0.f, 0.f, 0.f, 0.f}; });
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dyb[ks] = pack4(xs[2 * ks], xs[2 * ks + 1]);
        store_rows<C>(a.dy_row, dyb, t, a.T, g, c16);
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) xs[ft] = f32x4{0.f, 0.f, 0.f, 0.f};      // from here on: dn

        for (int j = 0; j < E; ++j) {
            u32x4 hb[KS], sl[KS], dtb[KS];
            {   // t_j, h_j and the slopes
                const uint8_t* wb = step_begin(3 * j);
                auto first = [&](auto act_c) {
                    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        f32x4 hv[2], sv[2];
#pragma unroll
                        for (int half = 0; half < 2; ++half) {
                            const int ft = 2 * ks + half;
                            f32x4 acc = *reinterpret_cast<const f32x4*>(pvec + j * C + 16 * ft + 4 * g);
#pragma unroll
                            for (int k2 = 0; k2 < KS; ++k2)
                                acc = M_::mma(*reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[k2]), nb[k2], acc);
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                float value, slope;
                                act_and_slope<ACT>(acc[r], value, slope);
                                hv[half][r] = value;
                                sv[half][r] = slope;
                            }
                        }
                        hb[ks] = pack4(hv[0], hv[1]);
                        sl[ks] = pack4(sv[0], sv[1]);
                    }
                };
                if (a.act == 0) first(std::integral_constant<int, 1>{}); else first(std::integral_constant<int, 2>{});
                store_rows<C>(a.a_in + (size_t)j * a.T * C, hb, t, a.T, g, c16);
                step_end();
            }
            {   // dh_j = W2[:,j]^T dy, dt_j = dh_j * act'(t_j)
                const uint8_t* wb = step_begin(3 * j + 1);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    f32x4 dv[2];
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const int ft = 2 * ks + half;
                        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int k2 = 0; k2 < KS; ++k2)
                            acc = M_::mma(*reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[k2]), dyb[k2], acc);
                        const uint32_t s0 = sl[ks][2 * half], s1 = sl[ks][2 * half + 1];
                        dv[half] = f32x4{acc[0] * M_::lo(s0), acc[1] * M_::hi(s0), acc[2] * M_::lo(s1), acc[3] * M_::hi(s1)};
                    }
                    dtb[ks] = pack4(dv[0], dv[1]);
                }
                store_rows<C>(a.g_out + (size_t)j * a.T * C, dtb, t, a.T, g, c16);
                step_end();
            }
            {   // dn += W1[j]^T dt_j
                const uint8_t* wb = step_begin(3 * j + 2);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    f32x4 acc = xs[ft];
#pragma unroll
                    for (int k2 = 0; k2 < KS; ++k2)
                        acc = M_::mma(*reinterpret_cast<const u32x4*>(wb + (16 * ft) * RS + woff[k2]), dtb[k2], acc);
                    xs[ft] = acc;
                }
                step_end();
            }
        }

        // ---- the norm's backward, dx (as in mlp_bwd_kernel) ----
        if (a.norm != 0) {
            u32x4 dq[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) dq[ks] = pack4(xs[2 * ks], xs[2 * ks + 1]);
            store_rows<C>(a.dn, dq, t, a.T, g, c16);
            if (live && lane < 16) *reinterpret_cast<float2*>(a.stats + 2 * tok) = make_float2(mean, rstd);
            float m1 = 0.f, m2 = 0.f;
            f32x4 xrow[FT];
            load_row<FT>(a.x, a.x_dtype, tok * a.xs + 4 * g, [&](int ft, f32x4 v) { xrow[ft] = v; });
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 xr = xrow[ft];
                const f32x4 gm = *reinterpret_cast<const f32x4*>(pvec + PG * C + 16 * ft + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    xs[ft][r] *= gm[r];
                    m1 += xs[ft][r];
                    m2 = fmaf(xs[ft][r], (xr[r] - mean) * rstd, m2);
                }
            }
            m1 = a.norm == 1 ? tok_sum(m1) * (1.f / C) : 0.f;
            m2 = tok_sum(m2) * (1.f / C);
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const f32x4 xr = xrow[ft];
#pragma unroll
                for (int r = 0; r < 4; ++r) xs[ft][r] = rstd * (xs[ft][r] - m1 - (xr[r] - mean) * rstd * m2);
            }
        }
        if (live) {
            if (a.add_dy & 1) {
                load_row<FT>(a.dy, a.dy_dtype, tok * a.dys + 4 * g, [&](int ft, f32x4 v) { xs[ft] += v; });
            }
            with_dtype(a.dx_dtype, [&](auto dc) {
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) st4(a.dx, tok * a.dxs + 16 * ft + 4 * g, decltype(dc)::value, xs[ft]);
            });
        }
    }
}

// dgamma[c] = sum_t ds_0[t,c] xhat[t,c],  dbeta[c] = sum_t ds_0[t,c]  over the workgroup's token range.  Thread =
// (group of four channels, token lane): 256 threads cover C / 4 groups x 1024 / C token lanes, every lane walks its
// tokens four at a time (all loads of a group in flight together: 16 bytes of x in fp32, 8 of ds_0), the lanes meet
// in LDS at the end.  One partial row pair per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void mlp_norm_grads_kernel(MlpBwdArgs a, int64_t tokens_per_wg)
{
    using M_ = Mw<T>;
    __shared__ f32x4 red[2][256];
    const int quads = a.C / 4, lanes = 256 / quads;             // 32 x 8, 16 x 16 or 8 x 32
    const int cq = threadIdx.x % quads, tl = threadIdx.x / quads;
    const int64_t t0 = (int64_t)blockIdx.x * tokens_per_wg, t1 = t0 + tokens_per_wg < a.T ? t0 + tokens_per_wg : a.T;
    f32x4 gs = {0.f, 0.f, 0.f, 0.f}, bs = {0.f, 0.f, 0.f, 0.f};
    for (int64_t t = t0 + tl; t < t1; t += 4 * lanes) {
        f32x4 xv[4];
        float2 st[4];
        uint2 dv[4];
        int64_t tt[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            tt[u] = t + u * lanes < t1 ? t + u * lanes : t1 - 1;
            st[u] = *reinterpret_cast<const float2*>(a.stats + 2 * tt[u]);
            dv[u] = *reinterpret_cast<const uint2*>(a.dn + (size_t)tt[u] * a.C + 4 * cq);
        }
        with_dtype(a.x_dtype, [&](auto dc) {        // one branch on the element type, the four loads back to back
            constexpr int DT = decltype(dc)::value;
            typename Raw4<DT>::type raw[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if constexpr (DT == 0) raw[u] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(a.x) + tt[u] * a.xs + 4 * cq);
                else raw[u] = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(a.x) + tt[u] * a.xs + 4 * cq);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) xv[u] = unpack4<DT>(raw[u]);
        });
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (t + u * lanes >= t1) continue;
            const f32x4 d = {M_::lo(dv[u].x), M_::hi(dv[u].x), M_::lo(dv[u].y), M_::hi(dv[u].y)};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                gs[r] = fmaf(d[r], (xv[u][r] - st[u].x) * st[u].y, gs[r]);
                bs[r] += d[r];
            }
        }
    }
    red[0][threadIdx.x] = gs;
    red[1][threadIdx.x] = bs;
    __syncthreads();
    if ((int)threadIdx.x < 2 * quads) {
        const int k = threadIdx.x / quads, q = threadIdx.x % quads;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        for (int l = 0; l < lanes; ++l) s += red[k][l * quads + q];
        *reinterpret_cast<f32x4*>(a.gb_part + ((size_t)blockIdx.x * 2 + k) * a.C + 4 * q) = s;
    }
}

// out[i] = sum over rows of part[row][i] (n = 2 C values per row).  A workgroup of 64 x 16 threads owns 64 values:
// thread (x, y) adds the rows y, y + 16, ... with eight loads in flight, the 16 y meet in LDS.  Fixed order.
__global__ __launch_bounds__(1024) void mlp_sum_rows_kernel(const float* part, int rows, int n, float* out)
{
    __shared__ float red[16][64];
    const int x = threadIdx.x & 63, y = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + x;
    float s = 0.f;
    if (i < n) {
        int r = y;
        for (; r + 112 < rows; r += 128) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(size_t)(r + 16 * u) * n + i];
            s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        }
        for (; r < rows; r += 16) s += part[(size_t)r * n + i];
    }
    red[y][x] = s;
    __syncthreads();
    if (y == 0 && i < n) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 16; ++k) t += red[k][x];
        out[i] = t;
    }
}

template <typename T, int C, int WAVES, int LMAX>
hipError_t launch_l(const MlpBwdArgs& a, hipStream_t st)
{
    auto kern = mlp_bwd_kernel<T, C, WAVES, LMAX>;
    const size_t wbuf = (size_t)C * C * 2;
    const size_t fixed = (size_t)(LMAX + 2) * C * sizeof(float);       // the kernel's own LDS array of parameter vectors
    int resident = (size_t)2 * a.L * wbuf + fixed <= 160 * 1024 ? 1 : 0;
    size_t lds = (resident ? (size_t)2 * a.L : 2) * wbuf;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess && resident) {
        (void)hipGetLastError();
        resident = 0;
        lds = 2 * wbuf;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    }
    if (e != hipSuccess) return e;
    const int64_t nblk = (a.T + WAVES * 16 - 1) / (WAVES * 16);
    const int64_t cus = device_cus();
    hipLaunchKernelGGL(kern, dim3((unsigned)(nblk < cus ? nblk : cus)), dim3(64 * WAVES), lds, st, a, resident);
    e = hipGetLastError();
    if (e != hipSuccess || a.norm == 0) return e;
    const int rows = mlp_bwd_partial_rows(a.T);
    const int64_t tpw = (a.T + rows - 1) / rows;
    hipLaunchKernelGGL(mlp_norm_grads_kernel<T>, dim3(rows), dim3(256), 0, st, a, tpw);
    e = hipGetLastError();
    if (e != hipSuccess || !a.gb) return e;
    hipLaunchKernelGGL(mlp_sum_rows_kernel, dim3((2 * C + 63) / 64), dim3(1024), 0, st, a.gb_part, rows, 2 * C, a.gb);
    return hipGetLastError();
}

// One workgroup per compute unit; its wave count is what the registers of the instance allow (two waves per SIMD
// up to 256 registers, three up to 168, four up to 128).
template <typename T, int C>
hipError_t launch_c(const MlpBwdArgs& a, hipStream_t st)
{
    if (a.L <= 1) return launch_l<T, C, (C == 128 ? 12 : 16), 1>(a, st);
    if (a.L <= 5) return launch_l<T, C, (C == 128 ? 8 : C == 64 ? 12 : 16), 5>(a, st);
    if (a.L <= mlp_bwd_max_layers(C)) return launch_l<T, C, (C == 32 ? 16 : 8), (C == 128 ? 5 : 8)>(a, st);
    return hipErrorInvalidValue;
}

template <typename T, int C, int WAVES>
hipError_t launch_expand(const MlpBwdArgs& a, hipStream_t st)
{
    auto kern = mlp_bwd_expand_kernel<T, C, WAVES>;
    const size_t lds = (size_t)2 * C * C * 2;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    const int64_t nblk = (a.T + WAVES * 16 - 1) / (WAVES * 16);
    const int64_t cus = device_cus();
    hipLaunchKernelGGL(kern, dim3((unsigned)(nblk < cus ? nblk : cus)), dim3(64 * WAVES), lds, st, a);
    e = hipGetLastError();
    if (e != hipSuccess || a.norm == 0) return e;
    const int rows = mlp_bwd_partial_rows(a.T);
    const int64_t tpw = (a.T + rows - 1) / rows;
    hipLaunchKernelGGL(mlp_norm_grads_kernel<T>, dim3(rows), dim3(256), 0, st, a, tpw);
    e = hipGetLastError();
    if (e != hipSuccess || !a.gb) return e;
    hipLaunchKernelGGL(mlp_sum_rows_kernel, dim3((2 * C + 63) / 64), dim3(1024), 0, st, a.gb_part, rows, 2 * C, a.gb);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_t(const MlpBwdArgs& a, hipStream_t st)
{
    if (a.E > 0) {
        if (a.E > kExpandMax) return hipErrorInvalidValue;
        switch (a.C) {
            case 32:  return launch_expand<T, 32, 16>(a, st);
            case 64:  return launch_expand<T, 64, 16>(a, st);
            case 128: return launch_expand<T, 128, 8>(a, st);
            default:  return hipErrorInvalidValue;
        }
    }
    switch (a.C) {
        case 32:  return launch_c<T, 32>(a, st);
        case 64:  return launch_c<T, 64>(a, st);
        case 128: return launch_c<T, 128>(a, st);
        default:  return hipErrorInvalidValue;
    }
}

}  // namespace

// layers whose activation slopes fit the registers of one lane
int mlp_bwd_max_layers(int C) { return C == 128 ? 5 : 8; }

// partial rows of dgamma, dbeta a launch writes (one per workgroup of the reduction over tokens: token ranges of at
// least 256 tokens, at most four workgroups per compute unit)
int mlp_bwd_partial_rows(int64_t T)
{
    const int64_t want = (T + 255) / 256, cap = 4 * (int64_t)device_cus();
    return (int)(want < cap ? (want < 1 ? 1 : want) : cap);
}

hipError_t launch_mlp_bwd(const MlpBwdArgs& a, int w_dtype, hipStream_t st)
{
    return w_dtype == 1 ? launch_t<bf16_t>(a, st) : launch_t<f16_t>(a, st);
}

}  // namespace flare
