// Shared device helpers and launch-argument structs for the gfx950 FLARE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace flare {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2   = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;  // "minus infinity" that stays finite under subtraction

// ---- element types -------------------------------------------------------------------
struct bf16_t { uint16_t x; };
typedef _Float16 f16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(uint32_t(v.x) << 16); }
__device__ __forceinline__ float to_f32(f16_t v) { return float(v); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40u);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                          // RNE
    return uint16_t(u >> 16);
}

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return bf16_t{f32_to_bf16_bits(v)}; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float v) { return f16_t(v); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The value of lane ^ 16 / lane ^ 32 with the row / half swaps of gfx950 (vector ALU, no LDS crossbar):
// swapping a register with its own copy leaves, in every lane, the lane's own value in one register of the
// pair and its partner's in the other.
typedef unsigned flare_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float sum_xor16(float x)
{
    const flare_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_xor32(float x)
{
    const flare_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float max_xor16(float x)
{
    const flare_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_xor32(float x)
{
    const flare_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// Counter-based keep/drop decision of attention dropout: a 24-bit hash of (seed, phase, b*H + h, latent, token);
// phase 0 = gather weights, 1 = scatter weights.  The backward recomputes it from the same inputs.
__host__ __device__ __forceinline__ uint32_t lowbias32(uint32_t x)
{
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}
__host__ __device__ __forceinline__ uint32_t dropout_hash24(uint32_t seed_lo, uint32_t seed_hi, uint32_t phase, uint32_t bh,
                                                            uint32_t m, uint32_t n)
{
    const uint32_t x = seed_lo + n * 0x9E3779B1u + m * 0x85EBCA77u + bh * 0xC2B2AE3Du + phase * 0x27D4EB2Fu;
    return lowbias32(lowbias32(x) ^ seed_hi) >> 8;
}

// Factor an entry of the softmax weights meets under attention dropout: 1 / (1 - p) if it is kept, 0 if not.
__device__ __forceinline__ float dropout_factor(uint32_t thr, float rs, uint32_t seed_lo, uint32_t seed_hi, uint32_t phase,
                                                uint32_t bh, uint32_t m, uint32_t n)
{
    return dropout_hash24(seed_lo, seed_hi, phase, bh, m, n) >= thr ? rs : 0.f;
}

// ---- kernel argument blocks (host fills them; passed by value) -------------------------
struct MixerArgs {
    const void* q; const void* k; const void* v; void* y;
    const uint8_t* mask;      // [B,N] or null
    float* z;                 // [B,H,M,D] fp32
    float* lse;               // [B,H,M] or null (natural log)
    float* lse_tok;           // [B,H,N] or null: natural log of each token's softmax sum over the latents (scatter)
    float* part_m;            // [B,H,P,M]   per-partial running max (log2 units)
    float* part_l;            // [B,H,P,M]   per-partial sum
    float* part_acc;          // [B,H,P,M,D] per-partial numerator
    int B, H, N, M, D;
    int n_splits;             // workgroups along N
    int n_parts;              // partials per (b,h): n_splits * partials-per-workgroup
    int tokens_per_split;
    float scale_log2;         // scale * log2(e)
    int no_mfma32;            // 1: keep the 16x16x32 kernels where the 32x32x16 ones would run
    int force_fma;            // 1: fp32 problems keep the FMA kernels (no fp32 matrix-core kernels)
    // attention dropout (not in the 32x32x16 kernels): an entry of the softmax weights is kept when its hash is >= drop_thr
    // (24-bit compare) and then scaled by drop_rs = 1 / (1 - p); drop_thr == 0 switches it off
    uint32_t drop_thr, seed_lo, seed_hi;
    float drop_rs;
    int64_t qs[3], ks[3], vs[3], ys[3];
};

struct CausalArgs {
    const void* q; const void* k; const void* v; void* y;
    float* mu; float* den; float* num;   // state, natural-log units for mu
    float* lse;                          // [B,H,N] or null: natural log of each token's softmax sum over the latents
    int* flags;                          // [B*H] or null: per-(b,h) "redo with the fp32 kernel" marks
    float* seg_den; float* seg_num;      // [B*H, n_slots, M] and [B*H, n_slots, M, D]: local states (matrix-core prefill)
    int n_segs, seg_len;                 // token segments processed in parallel; seg_len is a multiple of 16
    // First phase: tokens [0, (n_segs - 1) seg_len) cut into n_pieces pieces of piece_len tokens, one workgroup each
    // (so that this phase fills the device as evenly as the recurrence does, whatever n_segs - 1 is).  A piece writes
    // one local state per segment it touches; the slots are numbered in token order (causal_slot), and the last of the
    // n_slots slots stages the final state.
    int n_pieces, piece_len, n_slots;
    int B, H, N, M, D;
    int chunk;
    float scale;
    int64_t qs[3], ks[3], vs[3], ys[3];
};

// Segment boundaries b seg_len, b = 1..s, that fall inside a piece (not on a piece boundary): each of them splits a
// piece's tokens into two local states.
__host__ __device__ inline int causal_split_bounds(int s, int seg_len, int piece_len)
{
    int c = 0;
    for (int b = 1; b <= s; ++b) c += ((int64_t)b * seg_len) % piece_len != 0;
    return c;
}
// Slot of the local state of piece j's tokens inside segment s (the pair must exist), and the number of slots that
// hold tokens before segment `seg` (what its recurrence starts from, summed in slot order).
__host__ __device__ inline int causal_slot(int j, int s, int seg_len, int piece_len)
{
    return j + causal_split_bounds(s, seg_len, piece_len);
}
__host__ __device__ inline int causal_slots_before(int seg, int seg_len, int piece_len)
{
    if (seg <= 0) return 0;
    return (int)(((int64_t)seg * seg_len + piece_len - 1) / piece_len) + causal_split_bounds(seg - 1, seg_len, piece_len);
}

constexpr int kJoinMaxGroups = 16;
struct CausalJoinArgs {
    const void* yg[kJoinMaxGroups];      // per group: outputs [rows, D], contiguous, normalised within the group
    const float* lse[kJoinMaxGroups];    // per group: [rows] natural log of the group's softmax sum
    void* y;                             // [rows, D]
    int n_groups, D;
    int64_t rows;
};

struct TripleArgs {
    const void* q1; const void* q2; const void* k1; const void* k2; const void* v; void* out;
    float* state;      // [B,H,Dq,Dv,Dq]
    float* kk;         // [B,H,Dq,Dq] normaliser state or null
    float* part;       // [B,H,S,Dq*Dv*Dq (+Dq*Dq)] split partials
    int B, H, N, Dq, Dv;
    int feature_map, normalize;
    int diag_parts;    // 1: partials from the matrix-core kernel: blocks of 16^3 in accumulator order [step][lane][register]
    int n_splits, tokens_per_split;
    int n_parts;       // partials per (b,h) in `part`
    int64_t q1s[3], q2s[3], k1s[3], k2s[3], vs[3], os[3];
};

// Floats of one split partial of the triple state: [Dq][Dv][Dq] + [Dq][Dq] from the fp32 kernels, or one
// (16^3 + 16^2)-float tile per 16 x 16 x 16 block from the matrix-core kernels.
__host__ __device__ inline size_t triple_partial_floats(int Dq, int Dv, bool diag)
{
    return diag ? (size_t)(Dq / 16) * (Dv / 16) * (Dq / 16) * 4352 : (size_t)Dq * Dv * Dq + (size_t)Dq * Dq;
}

struct MixerBwdArgs {
    const void* q; const void* k; const void* v; const void* y; const void* dy;
    const float* z;          // [B,H,M,D] forward latent summary
    const float* lse_lat;    // [B,H,M] natural log of the gather's softmax sums
    const float* lse_tok;    // [B,H,N] natural log of the scatter's softmax sums
    float* delta_tok;        // [B,H,N]   <dy_n, y_n>               (workspace)
    float* dz;               // [B,H,M,D] gradient of z             (workspace)
    float* delta_lat;        // [B,H,M]   <dz_m, z_m>               (workspace)
    float* part;             // [B,H,P,M,D] split-N partial sums    (workspace)
    float* rho_min;          // [B,H,P]   smallest token log-sum-exp of each split, log2 units   (workspace)
    float* dq;               // [B,H,M,D] fp32
    void* dk; void* dv;      // [B,H,N,D] element type
    int B, H, N, M, D;
    int n_splits, tokens_per_split;      // split of the token axis a latent-side launch works in
    int n_splits0, tokens_per_split0;    // the dz pass's own split (rho_min has one entry per such split)
    float scale, scale_log2;
    int64_t qs[3], ks[3], vs[3], ys[3], dys[3], dks[3], dvs[3];
    int m0, mc, accumulate;  // token-side kernel only: latents [m0, m0 + mc) of the M (mc = 0: all), added to dk, dv when accumulate
    int scal_lds;            // token-side kernel only: per-latent scalars are tabled in LDS behind the operand sets
    int half;                // fp32 kernels: 0 = whole mixer, 1 = gather half only (dz given, no scatter term), 2 = scatter half only
                             // (no gather term, dv not written; dz is an output)
    int no_mfma32;           // 1: keep the 16x16x32 kernels where the 32x32x16 passes would run
    int only_form;           // token-side kernels: 0 = every (b,h); 1 = only those that take the unshifted one-exponential
                             // form (bwd_unshifted_form), 2 = only the others (a workgroup of the other kind returns at once)
    // attention dropout of the forward this is the backward of (same fields as MixerArgs; drop_thr == 0: none)
    uint32_t drop_thr, seed_lo, seed_hi;
    float drop_rs;
};

// Whether a (b,h) takes the form of the backward in which both weights come from exp2(S) alone (kernels on the 32x32x16
// product): the one-exponential form's own condition (the latents' largest log-sum-exp and the tokens' smallest one at
// most 64 apart, log2 units) and every latent log-sum-exp within +-60, so that exp2(S) can stand in for exp2(S - L2_m)
// with the constant exp2(-L2_m) applied elsewhere.  Every lane of a wave gets the same answer; lmax2 = largest L2_m.
__device__ __forceinline__ bool bwd_unshifted_form(const MixerBwdArgs& a, int64_t bh, int lane, float& lmax2)
{
    float lm = -3.0e38f, ln = 3.0e38f, rm = -3.0e38f;
    for (int m = lane; m < a.M; m += 64) {
        const float l = a.lse_lat[bh * a.M + m];
        lm = fmaxf(lm, l);
        ln = fminf(ln, l);
    }
    for (int p = lane; p < a.n_splits0; p += 64) rm = fmaxf(rm, -a.rho_min[bh * a.n_splits0 + p]);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        lm = fmaxf(lm, __shfl_xor(lm, o));
        ln = fminf(ln, __shfl_xor(ln, o));
        rm = fmaxf(rm, __shfl_xor(rm, o));
    }
    lmax2 = lm * kLog2e;
    return lmax2 <= 60.f && ln * kLog2e >= -60.f && lmax2 + rm <= 64.f;
}

struct CausalLinearArgs {
    const void* q; const void* k; const void* v; void* y;
    float* states;     // [B*H, n_segs, Dk, Dv] segment states (workspace)
    int B, H, N, Dk, Dv;
    int n_segs, seg_len;   // seg_len is a multiple of the 64-token tile
    float inv_n;           // 1 / N
    int64_t qs[3], ks[3], vs[3], ys[3];
};

struct MlpArgs {
    const void* x; const void* res; void* y;   // [T,C] rows; res may be null
    const uint16_t* w;                          // [L,C,C] 16-bit weights, row-major [out][in]
    const float* bias;                          // [L,C] or null
    const float* gamma; const float* beta;      // [C] norm parameters (beta may be null)
    int64_t T;
    int C, L;
    int x_dtype, res_dtype, y_dtype;            // 0 f32, 1 bf16, 2 f16
    int norm;                                   // 0 none, 1 LayerNorm, 2 RMSNorm
    float eps;
    int act;                                    // 0 tanh-GELU, 1 SiLU
    uint32_t act_mask, add_mask;                // bit l: layer l applies the activation / adds to the stream
    int expand;                                 // 1: L = 2E tiles of the two-layer MLP with hidden width E*C (see mlp_mfma.hip)
    int in_dim;                                 // > 0: x rows have in_dim <= 4 features and a first layer w_in lifts them to C
    const float* w_in;                          // [C][4] fp32 rows of the lifting layer (columns >= in_dim are zero), b_in [C]
    const float* b_in;
    int in_act;                                 // the lifting layer is followed by the activation
    int out_dim;                                // > 0: only features [0, out_dim <= 4) of the result are stored, y rows are out_dim wide
    int x_head, y_head;                         // > 0: rows of x / y hold heads of x_head / y_head (4 or 8) channels, each padded to 16 columns
    int64_t xs, rs, ys;                         // row strides in elements
};

// backward of the fused MLP chain (mlp_bwd_mfma.hip)
struct MlpBwdArgs {
    const void* x; const void* dy; void* dx;    // [T,C] rows: the forward's input, the gradient of its output, the gradient of x
    const uint16_t* w; const uint16_t* wt;      // [L,C,C] 16-bit weights [out][in] and their transposes [in][out]
    const float* bias;                          // [L,C] or null
    const float* gamma; const float* beta;      // [C] norm parameters (beta may be null)
    uint16_t* a_in;                             // [L,T,C] out: the input s_l of every layer, in the weights' type
    uint16_t* g_out;                            // [L,T,C] out: dt_l, the gradient at every layer's product, same type
    uint16_t* dn;                               // [T,C] out (norm != 0): ds_0, the gradient at the norm's output, same type
    float* stats;                               // [T,2] out (norm != 0): mean and 1/std of every token
    float* gb_part;                             // [rows,2,C] out (norm != 0): partial sums of dgamma, dbeta over token ranges
    float* gb;                                  // [2,C] out or null (norm != 0): the partial rows summed in index order
    int E;                                      // > 0: the expanding MLP C -> E C -> C (w, wt, bias hold 2 E tiles / rows;
    uint16_t* n_row; uint16_t* dy_row;          // a_in = h_j, g_out = dt_j per chunk; n and dy as 16-bit rows [T,C])
    int64_t T;
    int C, L;
    int x_dtype, dy_dtype, dx_dtype;            // 0 f32, 1 bf16, 2 f16
    int norm;                                   // 0 none, 1 LayerNorm, 2 RMSNorm
    float eps;
    int act;                                    // 0 tanh-GELU, 1 SiLU
    uint32_t act_mask, add_mask;
    int add_dy;                                 // bit 0: the forward's residual input was x itself, dx also receives dy; bit 1 (chain only): dx holds a gradient already and receives the sum
    int64_t xs, dys, dxs;                       // row strides in elements
};

// Arguments of the weight-gradient kernel (mlp_wgrad_mfma.hip): the rows launch_mlp_bwd leaves, reduced over tokens.
struct MlpWgradArgs {
    const uint16_t* a_in;                       // [L,T,C] the input of every layer (16-bit)
    const uint16_t* g_out;                      // [L,T,C] the gradient at every layer's product (16-bit)
    int64_t a_lstride, g_lstride;               // elements from one layer's rows to the next's (0: all layers share one array)
    float* dw_part;                             // [parts,L,C,C] out: partial dW_l[out][in] per token range
    float* db_part;                             // [parts,L,C] out or null: partial db_l
    float* dw; float* db;                       // [L,C,C], [L,C] out or null: the partials summed in index order
    int64_t T;
    int C, L;
    int64_t tokens_per_wg;                      // set by the launcher
};

// Workgroups of the backward's dq pass (bwd_lat_kernel, MODE 1) that fit a compute unit: its instances with 16 or
// 32 latents per wave at head dim 16, and with 16 at head dim 32, need few enough registers for three or four (measured:
// 143 -> 119 us at M = 128, D = 16; 86 -> 74 us at M = 64, D = 16; 133 -> 106 us at M = 64, D = 32); squeezing the
// others spills.  CT = 16-latent tiles per wave.
constexpr int bwd_dq_wgs_per_cu(int D, int CT)
{
    return D <= 16 ? (CT == 1 ? 4 : CT == 2 ? 3 : 2) : D <= 32 ? (CT == 1 ? 3 : 2) : 2;
}

// ---- launchers implemented in the .hip files -------------------------------------------
// dz pass of the mixer backward on the 32x32x16 product (mixer_bwd_mfma32.hip): bf16, D = 32, M % 64 == 0
bool       bwd_dz32_supported(int dtype, int M, int D);
hipError_t launch_bwd_dz32(const MixerBwdArgs& a, hipStream_t st);
int        bwd_dq32_mblocks(int M);
bool       bwd_tok32_supported(int dtype, int M, int D);
hipError_t launch_bwd_tok32(const MixerBwdArgs& a, hipStream_t st);      // only the (b,h) of the unshifted form
hipError_t launch_bwd_dq32(const MixerBwdArgs& a, hipStream_t st);
hipError_t launch_gather_generic(const MixerArgs& a, int dtype, hipStream_t st);
hipError_t launch_gather_merge(const MixerArgs& a, hipStream_t st);
hipError_t launch_scatter_generic(const MixerArgs& a, int dtype, hipStream_t st);
// fp32 inputs on v_mfma_f32_16x16x4_f32 (mixer_f32_mfma.hip): taken by the two launchers above when the problem allows
bool       f32_mfma_mixer_ok(const MixerArgs& a, bool scatter);
hipError_t launch_gather_f32_mfma(const MixerArgs& a, hipStream_t st);
hipError_t launch_scatter_f32_mfma(const MixerArgs& a, hipStream_t st);
int        gather_generic_parts_per_wg();

bool       mfma_mixer_supported(int dtype, int M, int D);
int        mfma_gather_tokens_per_iter(int dtype, int M, int D, bool allow32);
int        mfma_gather_resident_slots(int dtype, int M, int D, bool allow32);   // allow32: the 32x32x16 gather where it takes the shape
// workgroups of `kern` resident on the current device at once (CUs x occupancy), cached per kernel, LDS size and device
int        resident_slots(const void* kern, size_t dyn_lds, int block_threads = 256);
int        device_cus();
hipError_t launch_gather_mfma(const MixerArgs& a, int dtype, hipStream_t st);
hipError_t launch_scatter_mfma(const MixerArgs& a, int dtype, hipStream_t st);
// 32x32x16 instances (bf16, D = 32), chosen inside the two launchers above
bool       mfma32_gather_supported(int dtype, int M, int D, bool masked);
bool       mfma32_scatter_supported(int dtype, int M, int D, bool masked);
int        mfma32_gather_resident_slots(int M);
hipError_t launch_gather_mfma32(const MixerArgs& a, hipStream_t st);
hipError_t launch_scatter_mfma32(const MixerArgs& a, hipStream_t st);

size_t     causal_lds_bytes(int M, int D, bool decode);
hipError_t launch_causal_join(const CausalJoinArgs& a, int dtype, hipStream_t st);
hipError_t launch_causal_prefill(const CausalArgs& a, int dtype, hipStream_t st);
hipError_t launch_causal_decode(const CausalArgs& a, int dtype, hipStream_t st);
bool       causal_mfma_supported(int dtype, int M, int D);
hipError_t launch_causal_mfma(const CausalArgs& a, int dtype, int step, hipStream_t st);   // step 16 prefill, 1 decode
hipError_t launch_causal_decode_steps(const CausalArgs& a, int dtype, hipStream_t st);      // N one-token steps, same shapes as above

size_t     mixer_bwd_lds_bytes(int M, int D);
int        mixer_bwd_tok_chunks(int M, int D);
bool       mixer_bwd_supported(int dtype, int M, int D);
hipError_t launch_mixer_bwd(const MixerBwdArgs& a, int dtype, hipStream_t st);
// fp32 inputs on v_mfma_f32_16x16x4_f32 (mixer_bwd_f32_mfma.hip): D in {16, 32, 64}, M a multiple of 16
bool       mixer_bwd_f32_supported(int M, int D);
hipError_t launch_mixer_bwd_f32(const MixerBwdArgs& a, hipStream_t st);

bool       mlp_mfma_supported(int w_dtype, int C);
hipError_t launch_mlp_mfma(const MlpArgs& a, int w_dtype, hipStream_t st);
int        mlp_bwd_max_layers(int C);
int        mlp_bwd_partial_rows(int64_t T);
hipError_t launch_mlp_bwd(const MlpBwdArgs& a, int w_dtype, hipStream_t st);
int64_t    mlp_wgrad_tokens_per_wg(int64_t T, int C, int L);
int        mlp_wgrad_partials(int64_t T, int C, int L);
hipError_t launch_mlp_wgrad(const MlpWgradArgs& a, int w_dtype, hipStream_t st);

int        causal_linear_tile();
hipError_t launch_causal_linear(const CausalLinearArgs& a, int dtype, hipStream_t st);
hipError_t launch_causal_linear_prefix(const CausalLinearArgs& a, hipStream_t st);   // exclusive prefix over the segment states
// matrix-core kernels (causal_linear_mfma.hip): 16-bit inputs, Dk in {64, 128}, Dv in {32, 64, 128}
bool       causal_linear_mfma_supported(int dtype, int Dk, int Dv);
hipError_t launch_causal_linear_mfma(const CausalLinearArgs& a, int dtype, hipStream_t st);

hipError_t launch_triple_state(const TripleArgs& a, int dtype, hipStream_t st);
hipError_t launch_triple_merge(const TripleArgs& a, hipStream_t st);
hipError_t launch_triple_out(const TripleArgs& a, int dtype, hipStream_t st);
// fp32 inputs with head dims 16 on v_mfma_f32_16x16x4_f32 (triple_f32_mfma.hip): taken by the launchers above
bool       triple_f32_mfma_state_ok(const TripleArgs& a);
bool       triple_f32_mfma_out_ok(const TripleArgs& a);
hipError_t launch_triple_state_f32_mfma(const TripleArgs& a, hipStream_t st);
hipError_t launch_triple_out_f32_mfma(const TripleArgs& a, hipStream_t st);
bool       triple_mfma_supported(int dtype, int Dq, int Dv);
hipError_t launch_triple_state_mfma(const TripleArgs& a, int dtype, hipStream_t st);
hipError_t launch_triple_out_mfma(const TripleArgs& a, int dtype, hipStream_t st);

}  // namespace flare
