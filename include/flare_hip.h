/*
 * flare_hip.h — C-ABI of libflare_hip.so, the MI355X (gfx950) FLARE attention engine.
 *
 * Plain pointers and sizes only; no torch types.  Every device pointer is owned by the
 * caller (inputs, outputs and the workspace), with one exception: flare_mixer_fwd_static
 * works in a 64 MiB device array that is part of the library's code object, so every
 * process that loads the library holds those 64 MiB on each GPU it uses, whether or not it
 * calls that entry point.  The library calls no allocator (hipMalloc, hipFree), keeps no
 * mutable host state beyond a mutex-guarded cache of occupancy queries and of that array's
 * per-device address, launches asynchronously on the hipStream_t handed in (passed as
 * void*) and never synchronises the device.  All entry points return an int
 * status (0 = OK, negative = error); the text of the last error on the calling thread is
 * available from flare_last_error_string().  Shapes, dtypes, strides, alignment and the
 * workspace size are validated on the host BEFORE anything is launched.
 *
 * Reference interfaces each entry point replaces (paths relative to the reference tree):
 *   flare_mixer_fwd            README.md:39-52 (flare_multihead_mixer),
 *                              pdebench/models/flare.py:136-138, lra/models/backends.py:603-606
 *   flare_gather_fwd           first F.scaled_dot_product_attention(q, k, v) of the above
 *   flare_scatter_fwd          second F.scaled_dot_product_attention(k, q, z) of the above
 *   flare_scatter_fwd_lse      the same, also returning each token's log-sum-exp over the latents
 *   flare_gather_bwd / flare_scatter_bwd   gradients of the two calls above taken one at a time
 *   flare_mixer_bwd            gradient of flare_multihead_mixer (torch autograd through the two SDPA
 *                              calls upstream; ablation/time_memory_bwd.py:460-478 times fwd+bwd)
 *   flare_mixer_fwd_dropout    the same two calls with dropout_p > 0 (lra/models/backends.py:592,605-606)
 *   flare_mixer_fwd_static     (no counterpart upstream: flare_mixer_fwd without a caller workspace)
 *   flare_clock_probe          (no counterpart upstream: measurement aid, sustained shader clock)
 *   flare_causal_prefill_fwd   causal restriction of the mixer (README.md:60 names it; the
 *   flare_causal_decode_fwd    reference holds no code for it) following the 3-phase chunk
 *                              scheme of lra/models/triton/causal_linear.py:81-137 and the
 *                              token recurrence of causal_linear.py:317-336
 *   flare_causal_*_fwd_lse     the same with each token's log-sum-exp over the latents; flare_causal_join
 *                              combines latent groups with it (softmax over all latents = softmax over the
 *                              groups' sums times the softmax within each group)
 *   flare_causal_linear_fwd    CausalLinear.apply lra/models/triton/causal_linear.py:23-145
 *                              == linear_causal_reference causal_linear.py:317-336
 *   flare_mlp_fwd              ResidualMLP.forward pdebench/models/flare.py:45-59 (and lra/models/
 *                              backends.py:504-539), with the norm and residual around it of
 *                              FLAREBlock.forward flare.py:204-215; a chain of one layer is nn.Linear
 *   flare_triple_fwd           TripleAttentionFunction.apply lra/models/triton/triple.py:29-121
 *                              == TripleAttention.attn_einsum lra/models/backends.py:1285-1292
 */
#ifndef FLARE_HIP_H
#define FLARE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLARE_ABI_VERSION 2

/* status codes */
#define FLARE_OK            0
#define FLARE_EINVAL       (-1)  /* null pointer, bad shape / stride / alignment            */
#define FLARE_EUNSUPPORTED (-2)  /* valid request that no kernel covers (e.g. D > 128)      */
#define FLARE_EWORKSPACE   (-3)  /* workspace missing or smaller than *_workspace_bytes()   */
#define FLARE_EHIP         (-4)  /* a HIP runtime call failed (launch error)                */

/* element types of q / k / v / y */
#define FLARE_DT_F32  0
#define FLARE_DT_BF16 1
#define FLARE_DT_F16  2

/* FlareMixerDesc.flags */
#define FLARE_FLAG_FORCE_GENERIC 1  /* skip every matrix-core kernel (16-bit and fp32), use the fp32-FMA kernels */
#define FLARE_FLAG_MFMA16        2  /* keep the 16x16x32 MFMA kernels where the 32x32x16 gather and scatter (bf16, D = 32, no key mask) would run */
#define FLARE_FLAG_GRAD_LIKE_KV  8  /* flare_mixer_bwd: dk has k's strides and dv has v's (default: both [B,H,N,D] contiguous) */

/*
 * Mixer problem description.  Logical shapes:
 *   q [B?,H,M,D]   latent queries; q_stride[0] == 0 means one set shared by every batch
 *   k [B,H,N,D]    keys           v [B,H,N,D] values        y [B,H,N,D] output
 *   z [B,H,M,D]    latent summary, ALWAYS fp32 and contiguous
 * Strides are in ELEMENTS for dims (b, h, row); the innermost (D) stride must be 1, so
 * the [B,N,H*D] views produced by 'b n (h d) -> b h n d' are consumed without a copy.
 * Softmax and all accumulation are fp32 whatever the element type.
 */
typedef struct FlareMixerDesc {
    int32_t B, H, N, M, D;
    int32_t dtype;        /* FLARE_DT_* of q, k, v, y                                  */
    float   scale;        /* softmax scale s: scores are s * <q_m, k_n>                */
    int32_t n_splits;     /* gather split-N factor; 0 = choose automatically           */
    int32_t flags;        /* FLARE_FLAG_*                                              */
    int32_t reserved;
    int64_t q_stride[3];
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t y_stride[3];
    /* Attention dropout on both softmaxes, as torch's scaled_dot_product_attention applies it in training
     * (lra/models/backends.py:592,605-606: dropout_p on both calls): every normalised weight is kept with
     * probability 1 - dropout_p and then divided by it, independently in the gather and in the scatter.  The
     * decision for the weight of (batch, head, latent, token) is a counter-based hash of those indices, the phase
     * and dropout_seed compared with floor(dropout_p * 2^24) (no state, nothing stored): every entry point that
     * is handed the same descriptor sees the same mask, so the backward entry points regenerate the forward's.
     * 0 <= dropout_p < 1; 0 (and anything below 2^-24) switches dropout off.  Honoured by flare_gather_fwd,
     * flare_scatter_fwd(_lse), flare_mixer_fwd(_static) and flare_mixer_bwd; the 32x32x16 kernels carry no mask,
     * so a problem with dropout runs on the 16x16x32 (16-bit) or 16x16x4 (fp32) matrix-core kernels or on the
     * fp32-FMA kernels, and its workspace is sized from the descriptor with these fields set. */
    float    dropout_p;
    int32_t  reserved2;
    uint64_t dropout_seed;
} FlareMixerDesc;

/*
 * Causal FLARE.  Recurrent state per (b,h): mu[M] running max of s*<q_m,k_t>, den[M]
 * softmax denominator relative to mu, num[M,D] numerator relative to mu; all fp32,
 * contiguous [B,H,M], [B,H,M], [B,H,M,D].  A fresh state is mu=-inf (any value <= -1e30),
 * den=0, num=0.  For token t:
 *   sigma_m = s*<q_m,k_t>; mu' = max(mu, sigma); a = exp(mu-mu'); p = exp(sigma-mu');
 *   den = a*den + p; num = a*num + p (x) v_t; y_t = sum_m softmax_m(sigma)_m * num_m/den_m
 * k, v, y are [B,H,N,D] with the same stride convention as the mixer.
 */
typedef struct FlareCausalDesc {
    int32_t B, H, N, M, D;
    int32_t dtype;
    float   scale;
    int32_t chunk;        /* prefill segment length in tokens (rounded up to 16); 0 = automatic: the
                             token axis is cut so that about two workgroups per compute unit run,
                             segments of at least 256 tokens, at most 64 segments              */
    int32_t flags;
    int32_t reserved;
    int64_t q_stride[3];
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t y_stride[3];
} FlareCausalDesc;

/*
 * Triple (third-order) linear attention.  q1,q2,k1,k2 [B,H,N,Dq], v [B,H,N,Dv],
 *   state[b,h,i,j,k] = (1/N) sum_n f(k1)[n,i] v[n,j] f(k2)[n,k]      fp32 [B,H,Dq,Dv,Dq]
 *   out[b,h,n,j]     = sum_{i,k} f(q1)[n,i] state[i,j,k] f(q2)[n,k]  [B,H,N,Dv]
 * f = identity (feature_map 0) or elu(x)+1 (feature_map 1).  With normalize != 0 the
 * output is divided by the same contraction evaluated with v == 1.
 * All five inputs and out share one stride triple layout (b, h, n), innermost stride 1.
 */
typedef struct FlareTripleDesc {
    int32_t B, H, N, Dq, Dv;
    int32_t dtype;
    int32_t feature_map;  /* 0 identity, 1 elu+1 applied to q1,q2,k1,k2 inside the kernel */
    int32_t normalize;    /* 0 reference-exact (no denominator), 1 divide by normaliser  */
    int32_t n_splits;     /* state split-N factor; 0 = automatic                         */
    int32_t flags;
    int64_t q1_stride[3], q2_stride[3], k1_stride[3], k2_stride[3], v_stride[3], o_stride[3];
} FlareTripleDesc;

/*
 * Causal linear attention.  q, k [B,H,N,Dk], v, y [B,H,N,Dv] (Dk, Dv <= 128):
 *   y_t = (1/N) sum_{tau <= t} <q_t, k_tau> v_tau
 * (k and v each carry the reference's N^-1/2).  fp32 arithmetic whatever the element type.
 */
typedef struct FlareCausalLinearDesc {
    int32_t B, H, N, Dk, Dv;
    int32_t dtype;
    int32_t n_segs;       /* token segments processed in parallel; 0 = automatic          */
    int32_t flags;
    int64_t q_stride[3], k_stride[3], v_stride[3], y_stride[3];
} FlareCausalLinearDesc;

/*
 * Fused token-wise MLP stack:  s = norm(x);  for l < L: t = W_l s + b_l; t = act(t) if bit l of
 * act_mask; s = s + t if bit l of add_mask else t;  y = res + s.
 * x, res, y: [T, C] rows (row strides in elements, rows contiguous); w: [L, C, C] row-major
 * [out][in] in w_dtype (bf16 or f16, the type the products run in); bias [L, C], gamma, beta [C]
 * fp32.  ResidualMLP(C, C, C, n layers, input_residual, output_residual) is L = n + 2 with
 * act_mask = all but the last layer, add_mask = all layers (minus the first / last when the
 * matching flag is off).  C must be 32, 64 or 128.
 * With FLARE_MLP_EXPAND in flags the launch evaluates the two-layer MLP with hidden width E*C,
 * y = res + W2 act(W1 norm(x) + b1) + b2 (ResidualMLP(C, E*C, C, num_layers = 0), the "4x expansion"
 * feed-forward block), from L = 2E tiles of C x C weights in the order W1[0:C,:], W2[:,0:C],
 * W1[C:2C,:], W2[:,C:2C], ... and bias rows b1[0:C], b2, b1[C:2C], 0, ...; act_mask bit 0 says
 * whether the activation is applied, add_mask is ignored.
 */
#define FLARE_MLP_EXPAND 1
#define FLARE_NORM_NONE  0
#define FLARE_NORM_LAYER 1   /* (x - mean) * rsqrt(var + eps) * gamma + beta */
#define FLARE_NORM_RMS   2   /* x * rsqrt(mean(x^2) + eps) * gamma           */
#define FLARE_ACT_GELU_TANH 0
#define FLARE_ACT_SILU      1
typedef struct FlareMlpDesc {
    int64_t  T;
    int32_t  C, L;                        /* 1 <= L <= 16                                  */
    int32_t  w_dtype;                     /* FLARE_DT_BF16 or FLARE_DT_F16                 */
    int32_t  x_dtype, res_dtype, y_dtype; /* FLARE_DT_*                                    */
    int32_t  norm;                        /* FLARE_NORM_*                                  */
    float    eps;
    int32_t  act;                         /* FLARE_ACT_*                                   */
    uint32_t act_mask, add_mask;
    int32_t  flags;
    int64_t  x_stride, res_stride, y_stride;
} FlareMlpDesc;

int         flare_abi_version(void);
const char* flare_last_error_string(void);

/* Name of the kernel family the dispatcher would pick for this problem
 * ("mfma_bf16", "mfma_f16", "generic"); NULL + error on an invalid descriptor.  "generic" names the family that
 * serves fp32 and the shapes the 16-bit matrix-core kernels do not take: inside it, fp32 problems with D in
 * {16, 32, 64}, M a multiple of 16 and 16-byte aligned rows run on fp32 matrix-core kernels
 * (v_mfma_f32_16x16x4_f32), everything else as fp32 FMA loops; the workspace layout is the same for both. */
const char* flare_mixer_kernel_name(const FlareMixerDesc* desc);

/* Bytes of device workspace flare_gather_fwd / flare_mixer_fwd need for this problem. */
int flare_mixer_workspace_bytes(const FlareMixerDesc* desc, size_t* bytes);

/* z[B,H,M,D] (fp32) = softmax_n(s q k^T) v.  lse (fp32 [B,H,M], natural log of the softmax
 * normaliser) may be NULL.  key_mask (uint8 [B,N], 1 = token present) may be NULL; a
 * latent whose every key is masked gets z = 0. */
int flare_gather_fwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                     const uint8_t* key_mask, float* z, float* lse,
                     void* workspace, size_t workspace_bytes, void* stream);

/* y[B,H,N,D] = softmax_m(s k q^T) z.  Rows of masked tokens are written as 0. */
int flare_scatter_fwd(const FlareMixerDesc* desc, const void* q, const void* k, const float* z,
                      const uint8_t* key_mask, void* y, void* stream);

/* flare_scatter_fwd plus lse_tok (fp32 [B,H,N], may be NULL): natural log of sum_m exp(s <k_n,q_m>),
 * which the backward pass needs. */
int flare_scatter_fwd_lse(const FlareMixerDesc* desc, const void* q, const void* k, const float* z,
                          const uint8_t* key_mask, void* y, float* lse_tok, void* stream);

/* Backward of the mixer (bf16 / f16: D in {16,32,64}, M % 32 == 0, M D <= 65536; fp32: D in {16,32,64}, M % 16 == 0 -
 * the shapes flare_mixer_bwd_workspace_bytes accepts).  fp32 is the reference's default training precision
 * (pdebench/__main__.py:1106).  There is no key-mask
 * argument because none is needed: zero the k, v and dy rows of padded tokens, pass 1e30 as their lse_tok (and as
 * lse_lat of a batch element without tokens), and clear their dk, dv rows afterwards.
 * Inputs: q, k, v as in the forward; y and z its outputs; lse_lat = lse of flare_gather_fwd;
 * lse_tok of flare_scatter_fwd_lse; dy [B,H,N,D] with strides dy_stride.
 * Outputs: dq fp32 [B,H,M,D] contiguous (per batch element: sum over b when q is shared);
 * dk, dv [B,H,N,D] in the element type: contiguous, or with FLARE_FLAG_GRAD_LIKE_KV laid out as k and v are (a
 * projection that produced k token-major then takes dk back without a copy).
 * A forward that ran with desc->dropout_p > 0 is differentiated by handing the same descriptor (dropout_p and
 * dropout_seed) in here: the kernels regenerate its keep masks. */
int flare_mixer_bwd_workspace_bytes(const FlareMixerDesc* desc, size_t* bytes);
int flare_mixer_bwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v, const void* y,
                    const float* z, const float* lse_lat, const float* lse_tok, const void* dy,
                    const int64_t dy_stride[3], float* dq, void* dk, void* dv,
                    void* workspace, size_t workspace_bytes, void* stream);

/* Backward of the two halves called separately (same dtypes, shapes and workspace as flare_mixer_bwd, no dropout in
 * bf16 / f16; dk, dv in the element type, dy in the element type with strides that keep rows 16-byte aligned; models that
 * put layers between the halves: pdebench/models/flare_ablations.py:19-311 of the reference).  A key mask is handled
 * around them as for flare_mixer_bwd.
 * flare_gather_bwd:  gradient of flare_gather_fwd (the first scaled_dot_product_attention(q, k, v)): from dz
 *                    [B,H,M,D] fp32, with z and lse_lat of the forward, to dq [B,H,M,D] fp32, dk, dv [B,H,N,D].
 * flare_scatter_bwd: gradient of flare_scatter_fwd (the second scaled_dot_product_attention(k, q, z)): from dy, with y
 *                    and lse_tok of flare_scatter_fwd_lse, to dq, dk and dz [B,H,M,D] fp32 (the gradient of z). */
int flare_gather_bwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v, const float* z,
                     const float* lse_lat, const float* dz, float* dq, void* dk, void* dv,
                     void* workspace, size_t workspace_bytes, void* stream);
int flare_scatter_bwd(const FlareMixerDesc* desc, const void* q, const void* k, const float* z, const void* y,
                      const float* lse_tok, const void* dy, const int64_t dy_stride[3], float* dq, void* dk, float* dz,
                      void* workspace, size_t workspace_bytes, void* stream);

/* gather + merge + scatter on one stream.  z_out (fp32 [B,H,M,D]) may be NULL, in which
 * case z lives in the workspace. */
int flare_mixer_fwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                    const uint8_t* key_mask, void* y, float* z_out,
                    void* workspace, size_t workspace_bytes, void* stream);

/* flare_mixer_fwd with the descriptor's dropout fields taken from the arguments instead (desc->dropout_p and
 * desc->dropout_seed are ignored): the form lra/models/backends.py:592,605-606 calls, dropout_p on both softmaxes.
 * The workspace must hold flare_mixer_workspace_bytes() of the descriptor with dropout_p set. */
int flare_mixer_fwd_dropout(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                            const uint8_t* key_mask, float dropout_p, uint64_t seed, void* y, float* z_out,
                            void* workspace, size_t workspace_bytes, void* stream);

/* flare_mixer_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The split
 * partials and z live in a buffer of FLARE_STATIC_SCRATCH_BYTES that is part of the library's code object
 * (one copy per GPU, held until the process ends); the call allocates and frees nothing.  A problem whose
 * flare_mixer_workspace_bytes() exceeds that size is rejected with FLARE_EWORKSPACE before anything is
 * launched.  All calls on one GPU share the buffer: calls that overlap in time on the same GPU (different
 * streams or threads) race and must be serialised by the caller.  Results are those of flare_mixer_fwd.
 * Cost: the array is device memory of every process that has loaded the library, on every GPU that process
 * touches (16 processes sharing a GPU hold 1 GiB between them).  The first call on a device looks the
 * array's address up (hipGetSymbolAddress, which may load the code object): make that first call, with any
 * small problem, BEFORE a stream capture begins, since a lookup during capture can be refused; later calls
 * only launch kernels and may be captured. */
#define FLARE_STATIC_SCRATCH_BYTES (64u << 20)
int flare_mixer_fwd_static(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                           const uint8_t* key_mask, void* y, void* stream);

/* Diagnostic with no counterpart in the reference: one wave that reads the shader-clock counter and the
 * constant 100 MHz counter, sleeps for about `milliseconds` (at most 100) and reads both again.
 * out[0] = shader cycles, out[1] = 100 MHz ticks (device memory, two int64).  Launched on a second stream
 * beside the kernels under test it gives the clock the device actually sustains under their load, which is
 * what the matrix-core peak has to be scaled by (the device lowers its clock when matrix cores, vector units
 * and HBM all draw power). */
int flare_clock_probe(double milliseconds, int64_t* out, void* stream);

int flare_causal_workspace_bytes(const FlareCausalDesc* desc, size_t* bytes);

/* Chunked prefill over N tokens; state (mu, den, num) is read, advanced and written back. */
int flare_causal_prefill_fwd(const FlareCausalDesc* desc, const void* q, const void* k,
                             const void* v, void* y, float* mu, float* den, float* num,
                             void* workspace, size_t workspace_bytes, void* stream);

/* N recurrent single-token steps in ONE launch (desc->N = number of steps; k, v, y hold
 * the steps along their n axis); the state stays on chip between steps.  The workspace is
 * the one flare_causal_workspace_bytes() reports (it may be NULL when that is 0). */
int flare_causal_decode_fwd(const FlareCausalDesc* desc, const void* q, const void* k,
                            const void* v, void* y, float* mu, float* den, float* num,
                            void* workspace, size_t workspace_bytes, void* stream);

/* The same two entry points, also returning each token's log-sum-exp over the latents, lse_tok [B,H,N]
 * (natural log, contiguous): what joins latent groups that run as causal problems of their own. */
int flare_causal_prefill_fwd_lse(const FlareCausalDesc* desc, const void* q, const void* k,
                                 const void* v, void* y, float* lse_tok, float* mu, float* den, float* num,
                                 void* workspace, size_t workspace_bytes, void* stream);
int flare_causal_decode_fwd_lse(const FlareCausalDesc* desc, const void* q, const void* k,
                                const void* v, void* y, float* lse_tok, float* mu, float* den, float* num,
                                void* workspace, size_t workspace_bytes, void* stream);

/* Join of latent groups: y[r,:] = sum_g softmax_g(lse_groups[g][r]) * y_groups[g][r,:] over rows = B*H*N rows of
 * D elements (all contiguous, element type dtype, D a multiple of 8, at most FLARE_JOIN_MAX_GROUPS groups).
 * The softmax over all M latents of a token splits over groups of latents this way. */
#define FLARE_JOIN_MAX_GROUPS 16
int flare_causal_join(int32_t dtype, int32_t n_groups, int64_t rows, int32_t D, const void* const* y_groups,
                      const float* const* lse_groups, void* y, void* stream);

int flare_causal_linear_workspace_bytes(const FlareCausalLinearDesc* desc, size_t* bytes);

/* Segment states, exclusive prefix over the segments, then the outputs; sums in a fixed order.
 * Problems with Dk in {64, 128}, strides that are multiples of 8 elements and 16-byte aligned pointers run on the
 * matrix cores: bf16 / f16 with Dv in {32, 64, 128} (products in the input type, fp32 accumulation and state) and
 * fp32 with Dv in {32, 64} (fp32 products).  Everything else, and FLARE_FLAG_FORCE_GENERIC, as fp32 FMA loops. */
int flare_causal_linear_fwd(const FlareCausalLinearDesc* desc, const void* q, const void* k,
                            const void* v, void* y, void* workspace, size_t workspace_bytes,
                            void* stream);

/* bias, gamma (when norm == NONE), beta and res may be NULL.  y may alias res or x only row by
 * row at equal strides (every row is read completely before it is written). */
int flare_mlp_fwd(const FlareMlpDesc* desc, const void* x, const void* w, const float* bias,
                  const float* gamma, const float* beta, const void* res, void* y, void* stream);

/* The same stack between a narrow input and/or a narrow output (the models' in_proj and out_proj,
 * pdebench/models/flare.py:137-160: ResidualMLP(in_dim, C, C, ...) and ResidualMLP(C, C, out_dim, ...)).
 * in_dim > 0: x rows hold in_dim <= 4 features (x_stride >= in_dim, any alignment of the element
 *   type) and a first layer t = w_in x + b_in (w_in fp32 [C][4], columns >= in_dim zero; b_in fp32
 *   [C]; followed by the activation when in_act != 0) produces the stream the L tiles continue
 *   from; norm must be FLARE_NORM_NONE.  in_dim == 0: x rows are C wide as in flare_mlp_fwd.
 * out_dim > 0: only outputs [0, out_dim <= 4) of the last tile are stored (its other rows should be
 *   zero), y rows are out_dim wide (y_stride >= out_dim) and res must be NULL.  out_dim == 0: C wide.
 * Head-padded rows: FLARE_MLP_X_HEAD(h) / FLARE_MLP_Y_HEAD(h) in desc->flags (h = 4 or 8) say that
 *   the C channels of an x / y row are C/h heads of h channels and that each head occupies 16 columns of the row
 *   (channel f at column 16 (f / h) + f % h; x_stride / y_stride >= 16 C / h; stored pad columns are zeros).  This
 *   is the [B, N, H, 16] layout the mixer uses for head dims below 16.  Not combinable with in_dim / out_dim.  flare_mlp_fwd accepts these two flags as well.
 * FLARE_MLP_EXPAND is not accepted here. */
#define FLARE_MLP_X_HEAD(h) (((h) / 4) << 8)
#define FLARE_MLP_Y_HEAD(h) (((h) / 4) << 12)
int flare_mlp_io_fwd(const FlareMlpDesc* desc, int32_t in_dim, int32_t in_act, const float* w_in,
                     const float* b_in, int32_t out_dim, const void* x, const void* w, const float* bias,
                     const float* gamma, const float* beta, const void* res, void* y, void* stream);

#define FLARE_MLP_BWD_ADD_DY 1
#define FLARE_MLP_BWD_ACCUMULATE 2

/* Backward of flare_mlp_fwd for the chain of C x C layers (desc->flags == 0; at most 8 layers, 5 at C = 128): what
 * torch autograd computes for  y = res + ResidualMLP(norm(x))  (pdebench/models/flare.py:45-59, 204-215) when
 * the reference trains a block.  One token-parallel launch recomputes the forward and walks the chain back;
 * the reductions over all tokens that the weight and bias gradients need are a second call (flare_mlp_wgrad below):
 *   dx      [T,C]   contiguous, x's dtype: gradient of x.  add_dy is a set of bits: FLARE_MLP_BWD_ADD_DY = dy is
 *                   added (the forward's res was x itself; otherwise the gradient of res is dy);
 *                   FLARE_MLP_BWD_ACCUMULATE (this entry point only) = dx already holds a gradient of the same x, from
 *                   another chain that read it (the k and v projections of one block), and receives the sum -- what
 *                   autograd would otherwise add with a launch of its own
 *   a_in    [L,T,C] the input of every layer and
 *   g_out   [L,T,C] the gradient at every layer's product, both in the weights' type:
 *                   dW_l = g_out[l]^T a_in[l],  db_l = column sums of g_out[l]  (flare_mlp_wgrad forms both)
 *   dn      [T,C]   (norm only) gradient at the norm's output, weights' type;  stats [T,2] fp32 mean and 1/std
 *   gb_part [rows,2,C] fp32 (norm only; rows from flare_mlp_bwd_partial_rows): dgamma = sum over rows of
 *                   gb_part[:,0,:], dbeta = sum of gb_part[:,1,:] (fixed order: no atomics)
 *   gb      [2,C]   fp32 or NULL (norm only): those two sums, formed by one more small launch in index order
 * dy has desc->y_dtype and row stride desc->y_stride.  w_img, wt_img [L,C,C]: the weights and their transposes as
 * the kernel's LDS images: element (row, col) of a tile sits at 16-bit position
 *   row * C + 8 * (((4 * (ch / 4) + 2 * (ch % 2) + (j / 4)) ^ key)) + 4 * ((ch % 4) / 2) + j % 4,
 *   ch = col / 8, j = col % 8, key = (row % 16) >> (C == 128 ? 0 : C == 64 ? 1 : 2)
 * (flare.py_amd/fused.py::mlp_weight_image builds them). */
int flare_mlp_bwd_partial_rows(const FlareMlpDesc* desc, int32_t* rows);
/* Weight and bias gradients from the rows flare_mlp_bwd leaves, in one pass over both (the reference gets them from
 * torch's Linear backward: dW = dt^T s, db = column sums of dt; pdebench/models/flare.py:45-59 under autograd).
 * Only T, C, L and w_dtype of the descriptor are read.  a_in, g_out: L arrays of [T,C] rows in the weights' type,
 * a_layer_stride / g_layer_stride elements apart (T C when contiguous, 0 when all layers share one array);
 *   dw_part [parts,L,C,C] fp32: dW_l[out][in] = sum over parts of dw_part[:,l];
 *   db_part [parts,L,C]   fp32 or NULL: db_l = sum over parts of db_part[:,l]
 * with parts from flare_mlp_wgrad_partials;  dw [L,C,C], db [L,C] fp32 or NULL: those sums, formed by a second small
 * launch in index order (no atomics, two runs give the same bits). */
int flare_mlp_wgrad_partials(const FlareMlpDesc* desc, int32_t* parts);
int flare_mlp_wgrad(const FlareMlpDesc* desc, const void* a_in, int64_t a_layer_stride, const void* g_out, int64_t g_layer_stride,
                    float* dw_part, float* db_part, float* dw, float* db, void* stream);
/* Backward of flare_mlp_fwd with FLARE_MLP_EXPAND (y = res + W2 act(W1 norm(x) + b1) + b2, hidden width E C run as E
 * chunks; desc as for the forward: L = 2 E tiles, flags = FLARE_MLP_EXPAND; w_img, wt_img: LDS images of the 2 E tiles
 * and of their transposes, bias [2E,C] as for the forward).  Outputs as flare_mlp_bwd, with the rows for the weight
 * gradients arranged per chunk:
 *   n_row  [T,C]   norm(x) and  dy_row [T,C]  dy, both in the weights' type (shared by all chunks)
 *   h      [E,T,C] the hidden activations of every chunk,  dt [E,T,C] the gradient at the first product
 *   dW1[jC:(j+1)C, :] = dt[j]^T n_row,  db1[jC:(j+1)C] = column sums of dt[j]      (flare_mlp_wgrad, a stride 0)
 *   dW2[:, jC:(j+1)C] = dy_row^T h[j],   db2 = column sums of dy_row               (flare_mlp_wgrad, g stride 0) */
int flare_mlp_expand_bwd(const FlareMlpDesc* desc, const void* x, const void* dy, const void* w_img, const void* wt_img,
                         const float* bias, const float* gamma, const float* beta, int32_t add_dy, void* dx, void* n_row,
                         void* dy_row, void* h, void* dt, void* dn, float* stats, float* gb_part, float* gb, void* stream);
int flare_mlp_bwd(const FlareMlpDesc* desc, const void* x, const void* dy, const void* w_img, const void* wt_img,
                  const float* bias, const float* gamma, const float* beta, int32_t add_dy, void* dx, void* a_in,
                  void* g_out, void* dn, float* stats, float* gb_part, float* gb, void* stream);

int flare_triple_workspace_bytes(const FlareTripleDesc* desc, size_t* bytes);

/* state only (split-N partial sums + fixed-order merge; no atomics). */
int flare_triple_state_fwd(const FlareTripleDesc* desc, const void* k1, const void* k2,
                           const void* v, float* state, float* kk_state,
                           void* workspace, size_t workspace_bytes, void* stream);

/* out from a given state.  kk_state (fp32 [B,H,Dq,Dq]) is only read when normalize != 0. */
int flare_triple_out_fwd(const FlareTripleDesc* desc, const void* q1, const void* q2,
                         const float* state, const float* kk_state, void* out, void* stream);

/* state + out.  The workspace also holds kk_state when normalize != 0. */
int flare_triple_fwd(const FlareTripleDesc* desc, const void* q1, const void* q2,
                     const void* k1, const void* k2, const void* v, float* state, void* out,
                     void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLARE_HIP_H */
