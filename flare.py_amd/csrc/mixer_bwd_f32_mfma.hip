// Backward of the FLARE mixer for fp32 inputs on v_mfma_f32_16x16x4_f32 (the gradients torch autograd gives for
// README.md:39-52 of the reference; fp32 is the reference's default training precision, pdebench/__main__.py:1106).
//
// With the forward's two log-sum-exps (L_m of the gather, rho_n of the scatter) both weight matrices are plain
// exponentials of the scores, A[m,n] = exp(S - L_m) and B[n,m] = exp(S - rho_n), both <= 1, and
//   delta_n = <dy_n, y_n>          dz_m = sum_n B[n,m] dy_n          Delta_m = <dz_m, z_m>
//   dS[m,n] = A (<dz_m, v_n> - Delta_m) + B (<dy_n, z_m> - delta_n)
//   dv_n = sum_m A dz_m            dk_n = s sum_m dS q_m             dq_m = s sum_n dS k_n
// Three passes over the tokens, each shaped like one of the forward kernels of mixer_f32_mfma.hip (same operand
// conventions: A and B one float per lane, k-slot = lane group g, feature g D/4 + j in instruction j of a product over
// D; accumulator lane = column c16, rows 4g .. 4g + 3):
//   dz pass   (latent side, split over N)  dz partials, delta_n             -> merge: dz, Delta_m
//   token pass (token side)                dk, dv   (q, z, dz of the (b,h) in LDS)
//   dq pass   (latent side, split over N)  dq partials                      -> merge: dq
// The halves called separately (models with layers between them) run the same kernels with one term of dS dropped:
// the gather half takes dz from the caller, the scatter half returns it.
// Attention dropout of the forward (MixerBwdArgs::drop_thr != 0): its keep masks are regenerated from the same hash; with
// K the keep factors (0 or 1 / (1 - p)) the weights the forward used were K A and K B, so dz and dv meet K B and K A,
// and dS = A (K <dz, v> - Delta) + B (K <dy, z> - delta) with the same Delta and delta (they are sums over kept weights).
// Every sum has a fixed order: two runs give the same bits.  A key mask needs nothing here: the caller zeroes the
// padded tokens' rows and raises their log-sum-exp, so that their weights vanish.
#include <algorithm>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mma4(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f32x4 zero4f() { return f32x4{0.f, 0.f, 0.f, 0.f}; }

__device__ __forceinline__ float groups_sum(float x)
{
    x += __shfl_xor(x, 16);
    return x + __shfl_xor(x, 32);
}

// 16-latent tiles per wave of the latent-side passes
constexpr int lat_tiles(int D, int MODE) { return MODE == 1 && D == 64 ? 2 : 4; }

// a product over D of the rows the lanes hold: QL/4 chunks of four features each
template <int Q4> __device__ __forceinline__ f32x4 dot_rows(const f32x4 (&a)[Q4], const f32x4 (&b)[Q4])
{
    f32x4 s = zero4f();
#pragma unroll
    for (int j4 = 0; j4 < Q4; ++j4)
#pragma unroll
        for (int e = 0; e < 4; ++e) s = mma4(a[j4][e], b[j4][e], s);
    return s;
}

// ---- latent-side passes ----------------------------------------------------------------------------------------------
// One workgroup = 64 latents (32 in the dq pass at D = 64, whose three operand sets would not fit the registers) x one
// token range; wave w takes the 16-token tiles w, w + 4, ... of the range; the four
// waves' sums meet in LDS and the workgroup writes one partial [64][D].
// MODE 0: dz_m += B[n,m] dy_n (values = dY), and delta_n = <dy_n, y_n> from the first latent block.
// MODE 1: dq_m += dS[m,n] k_n (values = K), dS assembled from three score-like products.
template <int D, int MODE, int HALF, bool DROP>
__global__ __launch_bounds__(256, (D == 64 && MODE == 1) ? 1 : 2) void bwd_f32_lat_kernel(MixerBwdArgs a)
{
    constexpr int QL = D / 4, Q4 = QL / 4, RT = D / 16, VS = D + 4, VPT = D / 16;
    constexpr int CT = lat_tiles(D, MODE), MB = 16 * CT;      // latents per workgroup
    __shared__ __attribute__((aligned(16))) float vt[4][16][VS];     // the wave's value tile (dY or K), then the reduction

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int mblocks = (a.M + MB - 1) / MB;
    const int split = blockIdx.x / mblocks, mb = blockIdx.x % mblocks;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;
    const float* q = (const float*)a.q + b * a.qs[0] + h * a.qs[1];
    const float* k = (const float*)a.k + b * a.ks[0] + h * a.ks[1];
    const float* v = (const float*)a.v + b * a.vs[0] + h * a.vs[1];
    const float* y = (const float*)a.y + b * a.ys[0] + h * a.ys[1];
    const float* dy = (const float*)a.dy + b * a.dys[0] + h * a.dys[1];
    const float* lse_tok = a.lse_tok + bh * a.N;
    float* delta_tok = a.delta_tok + bh * a.N;
    const int tps = MODE == 0 ? a.tokens_per_split0 : a.tokens_per_split;
    const int n_parts = MODE == 0 ? a.n_splits0 : a.n_splits;
    constexpr bool use_a = HALF != 2, use_b = HALF != 1;      // gather term, scatter term of dS
    constexpr bool drop = DROP;                               // the forward dropped weights: the same masks are regenerated here

    // latent operands (B of the score-like products): q log2-scaled; for the dq pass also dz and z with their scalars
    f32x4 qb[CT][Q4], dzb[MODE ? CT : 1][Q4], zb[MODE ? CT : 1][Q4];
    float l2[CT], dl[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = mb * MB + 16 * ct + c16, mc = min(m, a.M - 1);
        const bool on = m < a.M;
#pragma unroll
        for (int j4 = 0; j4 < Q4; ++j4) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(q + (int64_t)mc * a.qs[2] + g * QL + 4 * j4);
            qb[ct][j4] = on ? t * a.scale_log2 : zero4f();
            if constexpr (MODE == 1) {
                const f32x4 t1 = *reinterpret_cast<const f32x4*>(a.dz + (bh * a.M + mc) * D + g * QL + 4 * j4);
                const f32x4 t2 = *reinterpret_cast<const f32x4*>(a.z + (bh * a.M + mc) * D + g * QL + 4 * j4);
                dzb[ct][j4] = on ? t1 : zero4f();
                zb[ct][j4] = on ? t2 : zero4f();
            }
        }
        l2[ct] = MODE ? a.lse_lat[bh * a.M + mc] * kLog2e : 0.f;
        dl[ct] = MODE ? a.delta_lat[bh * a.M + mc] : 0.f;
    }
    f32x4 acc[CT][RT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[ct][rt] = zero4f();

    const int n_begin = split * tps;
    const int n_end = min(a.N, n_begin + tps);
    const int tiles = n_begin < n_end ? (n_end - n_begin + 15) / 16 : 0;
    const int my_tiles = tiles > w ? (tiles - w + 3) / 4 : 0;

    // rows of the next tile, requested while this one is worked on (rows past the range repeat its last row)
    f32x4 ka[Q4], va[MODE ? Q4 : 1], dya[Q4], ya[MODE ? 1 : Q4], vr[VPT];
    float rho[4], dt[4];
    auto fetch = [&](int n0) {
        const int n = max(min(n0 + c16, n_end - 1), 0);
#pragma unroll
        for (int j4 = 0; j4 < Q4; ++j4) {
            ka[j4] = *reinterpret_cast<const f32x4*>(k + (int64_t)n * a.ks[2] + g * QL + 4 * j4);
            dya[j4] = *reinterpret_cast<const f32x4*>(dy + (int64_t)n * a.dys[2] + g * QL + 4 * j4);
            if constexpr (MODE == 1) va[j4] = *reinterpret_cast<const f32x4*>(v + (int64_t)n * a.vs[2] + g * QL + 4 * j4);
            else                     ya[j4] = *reinterpret_cast<const f32x4*>(y + (int64_t)n * a.ys[2] + g * QL + 4 * j4);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int nr = max(min(n0 + 4 * g + r, n_end - 1), 0);
            rho[r] = lse_tok[nr] * kLog2e;
            if constexpr (MODE == 1) dt[r] = delta_tok[nr];
        }
        // the value tile as it is written to LDS: dY rows (dz pass) or K rows (dq pass)
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = lane + 64 * i, tok = c / (D / 4), ch = c % (D / 4);
            const int nv = max(min(n0 + tok, n_end - 1), 0);
            vr[i] = MODE ? *reinterpret_cast<const f32x4*>(k + (int64_t)nv * a.ks[2] + 4 * ch)
                         : *reinterpret_cast<const f32x4*>(dy + (int64_t)nv * a.dys[2] + 4 * ch);
        }
    };
    int n0 = n_begin + 16 * w;
    if (my_tiles > 0) fetch(n0);
    for (int t = 0; t < my_tiles; ++t, n0 += 64) {
        f32x4 kc[Q4], vc[MODE ? Q4 : 1], dyc[Q4];
        float rh[4], de[4];
#pragma unroll
        for (int j4 = 0; j4 < Q4; ++j4) {
            kc[j4] = ka[j4];
            dyc[j4] = dya[j4];
            if constexpr (MODE == 1) vc[j4] = va[j4];
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            rh[r] = rho[r];
            de[r] = MODE ? dt[r] : 0.f;
        }
        // The tile passes between the lanes of the wave through LDS.  To the compiler every lane is a thread of its own: it
        // may move a lane's reads of other lanes' rows across that lane's own stores unless told not to.
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = lane + 64 * i, tok = c / (D / 4), ch = c % (D / 4);
            *reinterpret_cast<f32x4*>(&vt[w][tok][4 * ch]) = vr[i];
        }
        asm volatile("" ::: "memory");
        if constexpr (MODE == 0) if (mb == 0) {
            // delta_n = <dy_n, y_n>: the lane's share of the row, summed over the four lane groups
            float s = 0.f;
#pragma unroll
            for (int j4 = 0; j4 < Q4; ++j4)
#pragma unroll
                for (int e = 0; e < 4; ++e) s = fmaf(dya[j4][e], ya[j4][e], s);
            s = groups_sum(s);
            if (g == 0 && n0 + c16 < n_end) delta_tok[n0 + c16] = s;
        }
        bool valid[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) valid[r] = n0 + 4 * g + r < n_end;
        fetch(n0 + 64);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            // lane = latent column c16, rows = tokens 4g + r
            const f32x4 s = dot_rows<Q4>(kc, qb[ct]);
            float p[4];
            const uint32_t m_lat = (uint32_t)(mb * MB + 16 * ct + c16);
            if constexpr (MODE == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r) p[r] = valid[r] ? fast_exp2(s[r] - rh[r]) : 0.f;
                if constexpr (drop) {     // dz meets the scatter's weights as the forward applied them: kept ones, rescaled
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        p[r] *= dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 1u, (uint32_t)bh, m_lat, (uint32_t)(n0 + 4 * g + r));
                }
            } else {
                f32x4 t1 = dot_rows<Q4>(vc, dzb[ct]);      // <dz_m, v_n>
                f32x4 t2 = dot_rows<Q4>(dyc, zb[ct]);      // <dy_n, z_m>
                if constexpr (drop) {
                    // With W the weights and K the keep factors (0 or 1 / (1 - p)) the forward used K W, and the softmax
                    // gradient becomes W (K t - Delta): the inner products meet the keep factor, the row sums do not
                    // (Delta_m = <dz_m, z_m> and delta_n = <dy_n, y_n> already are the sums over the kept weights).
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t n = (uint32_t)(n0 + 4 * g + r);
                        if constexpr (use_a) t1[r] *= dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 0u, (uint32_t)bh, m_lat, n);
                        if constexpr (use_b) t2[r] *= dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 1u, (uint32_t)bh, m_lat, n);
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    // a half's absent term is left out at compile time: its operands may be anything
                    float ds = 0.f;
                    if constexpr (use_a) ds = fast_exp2(s[r] - l2[ct]) * (t1[r] - dl[ct]);
                    if constexpr (use_b) ds += fast_exp2(s[r] - rh[r]) * (t2[r] - de[r]);
                    p[r] = valid[r] ? ds : 0.f;
                }
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                f32x4 z = acc[ct][rt];
#pragma unroll
                for (int r = 0; r < 4; ++r) z = mma4(vt[w][4 * g + r][16 * rt + c16], p[r], z);    // acc^T[d, m] += X^T[d, n] P[n, m]
                acc[ct][rt] = z;
            }
        }
    }

    // the four waves' sums: every wave leaves its [64][D] block in LDS (its own value tile is dead by then), then
    // thread t adds the four copies of its elements in wave order
    __syncthreads();
    float* red = &vt[0][0][0];          // 4 * 16 * VS floats >= 64 * D / 4 per wave only for one quarter at a time
    const int64_t prow = ((bh * n_parts + split) * a.M);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        // quarter ct of the latents: [4 waves][16 latents][D]
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
            *reinterpret_cast<f32x4*>(red + (w * 16 + c16) * D + 16 * rt + 4 * g) = acc[ct][rt];
        __syncthreads();
        for (int e = tid; e < 16 * D; e += 256) {
            const float sum = (red[e] + red[16 * D + e]) + (red[32 * D + e] + red[48 * D + e]);
            const int m = mb * MB + 16 * ct + e / D;
            if (m < a.M) a.part[(prow + m) * D + e % D] = sum;
        }
        __syncthreads();
    }
}

// dz = sum of the split partials, Delta_m = <dz_m, z_m>  (MODE 0);  dq = scale * sum of the split partials  (MODE 1).
// One thread per (b, h, m); fixed order.
template <int MODE>
__global__ __launch_bounds__(256) void bwd_f32_merge_kernel(MixerBwdArgs a)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;      // (b*H + h)*M + m
    if (r >= (int64_t)a.B * a.H * a.M) return;
    const int64_t bh = r / a.M;
    const int m = (int)(r % a.M);
    const int P = MODE == 0 ? a.n_splits0 : a.n_splits;
    float delta = 0.f;
    for (int d = 0; d < a.D; d += 4) {
        f32x4 s = zero4f();
        for (int p = 0; p < P; ++p) s += *reinterpret_cast<const f32x4*>(a.part + ((bh * P + p) * a.M + m) * a.D + d);
        if (MODE == 0) {
            *reinterpret_cast<f32x4*>(a.dz + r * a.D + d) = s;
            const f32x4 zz = *reinterpret_cast<const f32x4*>(a.z + r * a.D + d);
            delta += s[0] * zz[0] + s[1] * zz[1] + s[2] * zz[2] + s[3] * zz[3];
        } else {
            *reinterpret_cast<f32x4*>(a.dq + r * a.D + d) = s * a.scale;
        }
    }
    if (MODE == 0) a.delta_lat[r] = delta;
}

// Delta_m = <dz_m, z_m> of a dz that the caller hands in (gather half): one thread per (b, h, m).
__global__ __launch_bounds__(256) void bwd_f32_delta_kernel(MixerBwdArgs a)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= (int64_t)a.B * a.H * a.M) return;
    float delta = 0.f;
    for (int d = 0; d < a.D; d += 4) {
        const f32x4 s = *reinterpret_cast<const f32x4*>(a.dz + r * a.D + d), zz = *reinterpret_cast<const f32x4*>(a.z + r * a.D + d);
        delta += s[0] * zz[0] + s[1] * zz[1] + s[2] * zz[2] + s[3] * zz[3];
    }
    a.delta_lat[r] = delta;
}

// ---- token pass: dk, dv ---------------------------------------------------------------------------------------------
// q (log2-scaled), z and dz rows of latents [m0, m0 + mc) of one (b,h) in LDS with their scalars; a wave takes 16 tokens
// at a time (lane = token column c16) and walks the latents 16 at a time (rows 4g + r).  8 waves per workgroup share
// the operands.  dk comes out in units of the log2-scaled q: multiplied by ln 2 at the end.
template <int D, int HALF>
__global__ __launch_bounds__(512) void bwd_f32_tok_kernel(MixerBwdArgs a)
{
    constexpr int QL = D / 4, Q4 = QL / 4, RT = D / 16, LS = D + 4;
    extern __shared__ __attribute__((aligned(16))) float smem_b[];
    const int MC = a.mc;
    float* qs = smem_b;                          // [MC][LS]
    float* zs = qs + (size_t)MC * LS;
    float* dzs = zs + (size_t)MC * LS;
    float* l2s = dzs + (size_t)MC * LS;          // [MC] latent log-sum-exp, log2 units
    float* dls = l2s + MC;                       // [MC] Delta_m

    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, c16 = lane & 15;
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t bh = (int64_t)b * a.H + h;
    const float* q = (const float*)a.q + b * a.qs[0] + h * a.qs[1];
    const float* k = (const float*)a.k + b * a.ks[0] + h * a.ks[1];
    const float* v = (const float*)a.v + b * a.vs[0] + h * a.vs[1];
    const float* dy = (const float*)a.dy + b * a.dys[0] + h * a.dys[1];
    float* dk = (float*)a.dk + b * a.dks[0] + h * a.dks[1];
    float* dv = (float*)a.dv + b * a.dvs[0] + h * a.dvs[1];
    const float* z = a.z + (bh * a.M + a.m0) * D;
    const float* dz = a.dz + (bh * a.M + a.m0) * D;

    for (int c = tid; c < MC * (D / 4); c += 512) {
        const int m = c / (D / 4), ch = c % (D / 4);
        *reinterpret_cast<f32x4*>(qs + m * LS + 4 * ch) = *reinterpret_cast<const f32x4*>(q + (int64_t)(a.m0 + m) * a.qs[2] + 4 * ch) * a.scale_log2;
        *reinterpret_cast<f32x4*>(zs + m * LS + 4 * ch) = *reinterpret_cast<const f32x4*>(z + (int64_t)m * D + 4 * ch);
        *reinterpret_cast<f32x4*>(dzs + m * LS + 4 * ch) = *reinterpret_cast<const f32x4*>(dz + (int64_t)m * D + 4 * ch);
    }
    for (int m = tid; m < MC; m += 512) {
        l2s[m] = a.lse_lat[bh * a.M + a.m0 + m] * kLog2e;
        dls[m] = a.delta_lat[bh * a.M + a.m0 + m];
    }
    __syncthreads();

    constexpr bool use_a = HALF != 2, use_b = HALF != 1;      // gather term, scatter term of dS
    const bool drop = a.drop_thr != 0;
    const int tiles = (a.N + 15) / 16;
    const int stride = gridDim.x * 8;
    int tile = blockIdx.x * 8 + w;
    const int my_tiles = tile < tiles ? (tiles - tile + stride - 1) / stride : 0;

    // K, V, dY rows as B operands straight from global memory, one tile ahead (rows past N repeat the last row)
    f32x4 kn[Q4], vn[Q4], dyn[Q4];
    float rho_n, delta_n;
    auto fetch = [&](int tl) {
        const int n = min(tl * 16 + c16, a.N - 1);
#pragma unroll
        for (int j4 = 0; j4 < Q4; ++j4) {
            kn[j4] = *reinterpret_cast<const f32x4*>(k + (int64_t)n * a.ks[2] + g * QL + 4 * j4);
            vn[j4] = *reinterpret_cast<const f32x4*>(v + (int64_t)n * a.vs[2] + g * QL + 4 * j4);
            dyn[j4] = *reinterpret_cast<const f32x4*>(dy + (int64_t)n * a.dys[2] + g * QL + 4 * j4);
        }
        rho_n = a.lse_tok[bh * a.N + n] * kLog2e;
        delta_n = a.delta_tok[bh * a.N + n];
    };
    if (my_tiles > 0) fetch(tile);
    for (int t = 0; t < my_tiles; ++t, tile += stride) {
        f32x4 kb[Q4], vb[Q4], dyb[Q4];
#pragma unroll
        for (int j4 = 0; j4 < Q4; ++j4) {
            kb[j4] = kn[j4];
            vb[j4] = vn[j4];
            dyb[j4] = dyn[j4];
        }
        const float rho = rho_n, dlt = delta_n;
        fetch(tile + stride);
        f32x4 dka[RT], dva[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) dka[rt] = dva[rt] = zero4f();
        for (int mt = 0; mt < MC / 16; ++mt) {
            // lane = token column c16, rows = latents 16 mt + 4g + r
            f32x4 qa[Q4], za[Q4], dza[Q4];
#pragma unroll
            for (int j4 = 0; j4 < Q4; ++j4) {
                qa[j4] = *reinterpret_cast<const f32x4*>(qs + (16 * mt + c16) * LS + g * QL + 4 * j4);
                za[j4] = *reinterpret_cast<const f32x4*>(zs + (16 * mt + c16) * LS + g * QL + 4 * j4);
                dza[j4] = *reinterpret_cast<const f32x4*>(dzs + (16 * mt + c16) * LS + g * QL + 4 * j4);
            }
            const f32x4 s = dot_rows<Q4>(qa, kb);
            f32x4 t1 = dot_rows<Q4>(dza, vb);       // <dz_m, v_n>
            f32x4 t2 = dot_rows<Q4>(za, dyb);       // <z_m, dy_n>
            const f32x4 l2 = *reinterpret_cast<const f32x4*>(l2s + 16 * mt + 4 * g);
            const f32x4 dl = *reinterpret_cast<const f32x4*>(dls + 16 * mt + 4 * g);
            float kf[4] = {1.f, 1.f, 1.f, 1.f};      // keep factors of the gather's weights (dv meets them too)
            if (drop) {
                const uint32_t n = (uint32_t)min(tile * 16 + c16, a.N - 1);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t m = (uint32_t)(a.m0 + 16 * mt + 4 * g + r);
                    if constexpr (use_a) {
                        kf[r] = dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 0u, (uint32_t)bh, m, n);
                        t1[r] *= kf[r];
                    }
                    if constexpr (use_b) t2[r] *= dropout_factor(a.drop_thr, a.drop_rs, a.seed_lo, a.seed_hi, 1u, (uint32_t)bh, m, n);
                }
            }
            float wa[4], ds[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // a half's absent term is left out at compile time: its operands may be anything
                wa[r] = 0.f;
                ds[r] = 0.f;
                if constexpr (use_a) {
                    const float wgt = fast_exp2(s[r] - l2[r]);
                    ds[r] = wgt * (t1[r] - dl[r]);
                    wa[r] = wgt * kf[r];
                }
                if constexpr (use_b) ds[r] += fast_exp2(s[r] - rho) * (t2[r] - dlt);
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                f32x4 o = dva[rt], u = dka[rt];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    o = mma4(dzs[(16 * mt + 4 * g + r) * LS + 16 * rt + c16], wa[r], o);     // dV^T[d, n] += dZ^T[d, m] A[m, n]
                    u = mma4(qs[(16 * mt + 4 * g + r) * LS + 16 * rt + c16], ds[r], u);      // dK^T[d, n] += Q^T[d, m] dS[m, n]
                }
                dva[rt] = o;
                dka[rt] = u;
            }
        }
        const int n = tile * 16 + c16;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the next tile's rows are waited for before the stores are issued
        if (n < a.N) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                f32x4* pk = reinterpret_cast<f32x4*>(dk + (int64_t)n * a.dks[2] + 16 * rt + 4 * g);
                f32x4* pv = reinterpret_cast<f32x4*>(dv + (int64_t)n * a.dvs[2] + 16 * rt + 4 * g);
                f32x4 ok = dka[rt] * kLn2, ov = dva[rt];
                if (a.accumulate) {
                    ok += *pk;
                    if constexpr (use_a) ov += *pv;
                }
                *pk = ok;
                if constexpr (use_a) *pv = ov;
            }
        }
    }
}

constexpr size_t kTokLdsMax = 150 * 1024;

// latents per launch of the token pass: three operand sets and two scalars per latent in LDS
int tok_chunk(int M, int D)
{
    const size_t per = (size_t)3 * (D + 4) * 4 + 8;
    int mc = (int)(kTokLdsMax / per) / 16 * 16;
    if (mc >= M) return M;
    const int chunks = (M + mc - 1) / mc;
    mc = ((M + chunks - 1) / chunks + 15) / 16 * 16;      // even chunks
    return mc;
}

template <int D, int HALF>
hipError_t launch_dh(const MixerBwdArgs& a0, hipStream_t st)
{
    MixerBwdArgs a = a0;
    const int mblocks = (a.M + 16 * lat_tiles(D, 0) - 1) / (16 * lat_tiles(D, 0)), mblocks1 = (a.M + 16 * lat_tiles(D, 1) - 1) / (16 * lat_tiles(D, 1));
    const int64_t rows = (int64_t)a.B * a.H * a.M;
    if (HALF == 1) {
        hipLaunchKernelGGL(bwd_f32_delta_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, a);
    } else {
        if (a.drop_thr != 0) hipLaunchKernelGGL((bwd_f32_lat_kernel<D, 0, 0, true>), dim3(a.n_splits0 * mblocks, a.H, a.B), dim3(256), 0, st, a);
        else                 hipLaunchKernelGGL((bwd_f32_lat_kernel<D, 0, 0, false>), dim3(a.n_splits0 * mblocks, a.H, a.B), dim3(256), 0, st, a);
        hipLaunchKernelGGL(bwd_f32_merge_kernel<0>, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, a);
    }
    // token pass, in chunks of latents when their operands do not fit the LDS
    const int mc = tok_chunk(a.M, D);
    auto kern = bwd_f32_tok_kernel<D, HALF>;
    const size_t lds = (size_t)mc * ((size_t)3 * (D + 4) * 4 + 8);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    const int64_t groups = ((int64_t)a.N + 127) / 128;
    // two rounds of the device (one workgroup of eight waves per compute unit at a time)
    const int64_t want = std::max<int64_t>(1, ((int64_t)2 * device_cus() + (int64_t)a.B * a.H - 1) / ((int64_t)a.B * a.H));
    const dim3 grid((unsigned)std::min<int64_t>(groups, want), a.H, a.B);
    for (int m0 = 0; m0 < a.M; m0 += mc) {
        a.m0 = m0;
        a.mc = std::min(mc, a.M - m0);
        a.accumulate = m0 > 0;
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, a);
    }
    if (a.drop_thr != 0) hipLaunchKernelGGL((bwd_f32_lat_kernel<D, 1, HALF, true>), dim3(a.n_splits * mblocks1, a.H, a.B), dim3(256), 0, st, a);
    else                 hipLaunchKernelGGL((bwd_f32_lat_kernel<D, 1, HALF, false>), dim3(a.n_splits * mblocks1, a.H, a.B), dim3(256), 0, st, a);
    hipLaunchKernelGGL(bwd_f32_merge_kernel<1>, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, a);
    return hipGetLastError();
}

template <int D>
hipError_t launch_d(const MixerBwdArgs& a, hipStream_t st)
{
    return a.half == 1 ? launch_dh<D, 1>(a, st) : a.half == 2 ? launch_dh<D, 2>(a, st) : launch_dh<D, 0>(a, st);
}

}  // namespace

bool mixer_bwd_f32_supported(int M, int D)
{
    return (D == 16 || D == 32 || D == 64) && M >= 16 && M % 16 == 0;
}

hipError_t launch_mixer_bwd_f32(const MixerBwdArgs& a, hipStream_t st)
{
    switch (a.D) {
        case 16: return launch_d<16>(a, st);
        case 32: return launch_d<32>(a, st);
        case 64: return launch_d<64>(a, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace flare
