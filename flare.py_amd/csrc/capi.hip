// extern "C" boundary of libflare_hip.so: host-side validation, planning and dispatch.
// No exception crosses this file; every error is a status code plus a thread-local text.
#include "../../include/flare_hip.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "common.hpp"

// Scratch memory of flare_mixer_fwd_static: one array per device, held until the process ends.  Its name is
// only a host-side handle; the device address is looked up once per device (static_scratch below).
static __device__ __align__(256) unsigned char scratch[FLARE_STATIC_SCRATCH_BYTES];

static_assert(FLARE_JOIN_MAX_GROUPS == flare::kJoinMaxGroups, "header and kernel argument block disagree");

namespace {

// One wave: shader cycles and 100 MHz ticks that pass while it sleeps for `ticks` of the 100 MHz counter.
// The loop is bounded by that counter, which never stops, so the wave always exits.
__global__ void clock_probe_kernel(long long* out, long long ticks)
{
    const long long r0 = wall_clock64(), c0 = clock64();
    while (wall_clock64() - r0 < ticks) __builtin_amdgcn_s_sleep(64);
    const long long c1 = clock64(), r1 = wall_clock64();
    if (threadIdx.x == 0) {
        out[0] = c1 - c0;
        out[1] = r1 - r0;
    }
}

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int esize(int dtype) { return dtype == FLARE_DT_F32 ? 4 : 2; }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

bool strides_mult8(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }

// ---- mixer ----------------------------------------------------------------------------
struct MixerPlan {
    bool mfma;
    int n_splits, n_parts, tokens_per_split;
    size_t off_m, off_l, off_acc, off_z, total;
};

int check_mixer_desc(const FlareMixerDesc* d)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->B < 1 || d->H < 1 || d->N < 1 || d->M < 1 || d->D < 1)
        return fail(FLARE_EINVAL, "B,H,N,M,D must be >= 1 (got %d,%d,%d,%d,%d)", d->B, d->H, d->N, d->M, d->D);
    if (d->dtype < FLARE_DT_F32 || d->dtype > FLARE_DT_F16) return fail(FLARE_EINVAL, "unknown dtype %d", d->dtype);
    if (!(d->scale > 0.f)) return fail(FLARE_EINVAL, "scale must be > 0 (got %g)", (double)d->scale);
    if (d->D > 128) return fail(FLARE_EUNSUPPORTED, "head dim D=%d > 128 is not supported", d->D);
    if (d->H > 65535 || d->B > 65535) return fail(FLARE_EUNSUPPORTED, "B and H must be <= 65535");
    if (d->n_splits < 0) return fail(FLARE_EINVAL, "n_splits must be >= 0");
    if (!(d->dropout_p >= 0.f) || !(d->dropout_p < 1.f)) return fail(FLARE_EINVAL, "dropout_p must be in [0, 1) (got %g)", (double)d->dropout_p);
    const int64_t* ss[4] = {d->q_stride, d->k_stride, d->v_stride, d->y_stride};
    const char* nm[4] = {"q", "k", "v", "y"};
    for (int t = 0; t < 4; ++t) {
        if (ss[t][2] < d->D) return fail(FLARE_EINVAL, "%s row stride %lld < D=%d (rows overlap)", nm[t], (long long)ss[t][2], d->D);
        if (ss[t][0] < 0 || ss[t][1] < 0) return fail(FLARE_EINVAL, "%s has a negative stride", nm[t]);
    }
    return FLARE_OK;
}

bool mixer_ptrs_ok_for_mfma(const FlareMixerDesc* d, const void* q, const void* k, const void* v, const void* y)
{
    if (q && !aligned16(q)) return false;
    if (k && !aligned16(k)) return false;
    if (v && !aligned16(v)) return false;
    if (y && !aligned16(y)) return false;
    return strides_mult8(d->q_stride) && strides_mult8(d->k_stride) && strides_mult8(d->v_stride) &&
           strides_mult8(d->y_stride);
}

// 24-bit threshold of the keep/drop hash: an entry is dropped when its hash is below it.  0 = no dropout (also for a
// dropout_p below 2^-24, which keeps every weight and rescales nothing).
uint32_t drop_threshold(const FlareMixerDesc* d) { return (uint32_t)((double)d->dropout_p * 16777216.0); }

// The plan depends on the descriptor only (never on pointer values) so that the workspace
// query and the launch always agree.  Misaligned pointers demote to the generic kernels,
// whose partial count (4 per workgroup) is covered by sizing for the larger of the two.
MixerPlan plan_mixer(const FlareMixerDesc* d, bool want_mfma)
{
    MixerPlan p;
    p.mfma = want_mfma;
    const bool allow32 = !(d->flags & FLARE_FLAG_MFMA16) && drop_threshold(d) == 0;     // the 32x32x16 kernels carry no dropout
    const int unit = p.mfma ? flare::mfma_gather_tokens_per_iter(d->dtype, d->M, d->D, allow32) : 32;
    const int mblk = p.mfma ? ((d->M % 256 == 0 && d->D <= 32) ? d->M / 256 : (d->M % 128 == 0) ? d->M / 128 : (d->M + 63) / 64)
                            : (d->M + 63) / 64;
    int s = d->n_splits;
    if (s <= 0) {
        // one full round of resident workgroups (MFMA kernels) or ~4 per CU (generic)
        const int64_t target = p.mfma ? flare::mfma_gather_resident_slots(d->dtype, d->M, d->D, allow32) : 4 * flare::device_cus();
        int64_t per = (int64_t)d->B * d->H * mblk;
        s = (int)((target + per - 1) / per);
        if (s < 1) s = 1;
    }
    int64_t tps = ((int64_t)d->N + s - 1) / s;
    tps = ((tps + unit - 1) / unit) * unit;
    const int min_tokens = p.mfma ? 4 * unit : 8 * unit;  // keep the split overhead small
    if (tps < min_tokens) tps = min_tokens;
    p.tokens_per_split = (int)tps;
    p.n_splits = (int)(((int64_t)d->N + tps - 1) / tps);
    p.n_parts = p.mfma ? p.n_splits : p.n_splits * flare::gather_generic_parts_per_wg();
    const size_t bh = (size_t)d->B * d->H;
    const size_t rows = bh * p.n_parts * d->M;
    p.off_m = 0;
    p.off_l = p.off_m + rows * 4;
    p.off_acc = p.off_l + rows * 4;
    p.off_z = p.off_acc + rows * d->D * 4;
    p.off_z = (p.off_z + 255) & ~(size_t)255;
    p.total = p.off_z + bh * d->M * d->D * 4;
    return p;
}

bool desc_wants_mfma(const FlareMixerDesc* d)
{
    return !(d->flags & FLARE_FLAG_FORCE_GENERIC) && flare::mfma_mixer_supported(d->dtype, d->M, d->D) &&
           strides_mult8(d->q_stride) && strides_mult8(d->k_stride) && strides_mult8(d->v_stride) &&
           strides_mult8(d->y_stride);
}

size_t mixer_ws_bytes(const FlareMixerDesc* d)
{
    size_t a = plan_mixer(d, false).total;
    if (desc_wants_mfma(d)) {
        size_t b = plan_mixer(d, true).total;
        if (b > a) a = b;
    }
    return a;
}

void fill_mixer_args(flare::MixerArgs& a, const FlareMixerDesc* d, const MixerPlan& p, void* ws)
{
    memset(&a, 0, sizeof(a));
    a.B = d->B; a.H = d->H; a.N = d->N; a.M = d->M; a.D = d->D;
    a.n_splits = p.n_splits; a.n_parts = p.n_parts; a.tokens_per_split = p.tokens_per_split;
    a.scale_log2 = d->scale * flare::kLog2e;
    a.no_mfma32 = (d->flags & FLARE_FLAG_MFMA16) ? 1 : 0;
    a.force_fma = (d->flags & FLARE_FLAG_FORCE_GENERIC) ? 1 : 0;
    a.drop_thr = drop_threshold(d);
    a.drop_rs = 1.f;
    if (a.drop_thr != 0) {
        a.no_mfma32 = 1;
        a.drop_rs = 1.0f / (1.0f - d->dropout_p);
        a.seed_lo = (uint32_t)(d->dropout_seed & 0xffffffffu);
        a.seed_hi = (uint32_t)(d->dropout_seed >> 32);
    }
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = d->q_stride[i]; a.ks[i] = d->k_stride[i]; a.vs[i] = d->v_stride[i]; a.ys[i] = d->y_stride[i];
    }
    if (ws) {
        char* w = static_cast<char*>(ws);
        a.part_m = reinterpret_cast<float*>(w + p.off_m);
        a.part_l = reinterpret_cast<float*>(w + p.off_l);
        a.part_acc = reinterpret_cast<float*>(w + p.off_acc);
    }
}

int hip_status(hipError_t e, const char* what)
{
    if (e == hipSuccess) return FLARE_OK;
    return fail(FLARE_EHIP, "%s: %s", what, hipGetErrorString(e));
}

int do_gather(const FlareMixerDesc* d, const void* q, const void* k, const void* v, const uint8_t* mask,
              float* z, float* lse, void* ws, size_t ws_bytes, hipStream_t st)
{
    if (!ws) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    if (!aligned16(ws)) return fail(FLARE_EINVAL, "workspace must be 16-byte aligned");
    const size_t need = mixer_ws_bytes(d);
    if (ws_bytes < need) return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", ws_bytes, need);
    const bool mfma = desc_wants_mfma(d) && mixer_ptrs_ok_for_mfma(d, q, k, v, nullptr);
    const MixerPlan p = plan_mixer(d, mfma);
    flare::MixerArgs a;
    fill_mixer_args(a, d, p, ws);
    a.q = q; a.k = k; a.v = v; a.mask = mask; a.z = z; a.lse = lse;
    hipError_t e = mfma ? flare::launch_gather_mfma(a, d->dtype, st) : flare::launch_gather_generic(a, d->dtype, st);
    if (e != hipSuccess) return hip_status(e, "gather launch");
    return hip_status(flare::launch_gather_merge(a, st), "gather merge launch");
}

int do_scatter(const FlareMixerDesc* d, const void* q, const void* k, const float* z, const uint8_t* mask,
               void* y, hipStream_t st, float* lse_tok = nullptr)
{
    const bool mfma = desc_wants_mfma(d) && mixer_ptrs_ok_for_mfma(d, q, k, nullptr, y);
    const MixerPlan p = plan_mixer(d, mfma);
    flare::MixerArgs a;
    fill_mixer_args(a, d, p, nullptr);
    a.q = q; a.k = k; a.y = y; a.mask = mask; a.z = const_cast<float*>(z); a.lse_tok = lse_tok;
    hipError_t e = mfma ? flare::launch_scatter_mfma(a, d->dtype, st) : flare::launch_scatter_generic(a, d->dtype, st);
    return hip_status(e, "scatter launch");
}

// ---- causal ---------------------------------------------------------------------------
int check_causal_desc(const FlareCausalDesc* d)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->B < 1 || d->H < 1 || d->N < 1 || d->M < 1 || d->D < 1)
        return fail(FLARE_EINVAL, "B,H,N,M,D must be >= 1 (got %d,%d,%d,%d,%d)", d->B, d->H, d->N, d->M, d->D);
    if (d->dtype < FLARE_DT_F32 || d->dtype > FLARE_DT_F16) return fail(FLARE_EINVAL, "unknown dtype %d", d->dtype);
    if (!(d->scale > 0.f)) return fail(FLARE_EINVAL, "scale must be > 0 (got %g)", (double)d->scale);
    if (d->D > 128) return fail(FLARE_EUNSUPPORTED, "head dim D=%d > 128 is not supported", d->D);
    if (d->chunk < 0) return fail(FLARE_EINVAL, "chunk must be >= 0");
    if (flare::causal_lds_bytes(d->M, d->D, false) > 160 * 1024)
        return fail(FLARE_EUNSUPPORTED, "state M*D=%d*%d does not fit the 160 KB LDS", d->M, d->D);
    if ((int64_t)d->B * d->H > 2147483647LL / 4) return fail(FLARE_EUNSUPPORTED, "B*H too large");
    const int64_t* ss[4] = {d->q_stride, d->k_stride, d->v_stride, d->y_stride};
    const char* nm[4] = {"q", "k", "v", "y"};
    for (int t = 0; t < 4; ++t)
        if (ss[t][2] < d->D) return fail(FLARE_EINVAL, "%s row stride %lld < D=%d", nm[t], (long long)ss[t][2], d->D);
    return FLARE_OK;
}

bool causal_wants_mfma(const FlareCausalDesc* d)
{
    return !(d->flags & FLARE_FLAG_FORCE_GENERIC) && flare::causal_mfma_supported(d->dtype, d->M, d->D) &&
           strides_mult8(d->q_stride) && strides_mult8(d->k_stride) && strides_mult8(d->v_stride) &&
           strides_mult8(d->y_stride);
}

// Matrix-core prefill plan: the token axis is cut into segments that run in parallel (local
// states first, then the recurrence of each segment from the summed states before it).
struct CausalPlan { bool mfma; int n_segs, seg_len, n_pieces, piece_len, n_slots; size_t off_den, off_num, total; };

CausalPlan plan_causal(const FlareCausalDesc* d)
{
    CausalPlan p{};
    p.mfma = causal_wants_mfma(d);
    p.n_segs = 1;
    p.seg_len = d->N;
    if (!p.mfma) return p;
    const int64_t BH = (int64_t)d->B * d->H;
    int64_t seg_len;
    if (d->chunk > 0) {
        seg_len = ((int64_t)d->chunk + 15) / 16 * 16;
    } else {
        // two workgroups per compute unit (what the kernel's LDS footprint allows), segments of at least 256 tokens
        const int64_t want = std::max<int64_t>(1, (2 * flare::device_cus() + BH - 1) / BH);
        seg_len = std::max<int64_t>(256, ((d->N + want - 1) / want + 15) / 16 * 16);
    }
    int64_t n_segs = (d->N + seg_len - 1) / seg_len;
    if (n_segs > 64) {
        seg_len = ((d->N + 63) / 64 + 15) / 16 * 16;
        n_segs = (d->N + seg_len - 1) / seg_len;
    }
    p.n_pieces = 0;
    p.piece_len = (int)seg_len;
    p.n_slots = 1;
    if (n_segs > 1) {
        p.n_segs = (int)n_segs;
        p.seg_len = (int)seg_len;
        // The first phase covers the tokens before the last segment.  With one workgroup per segment it would run
        // n_segs - 1 workgroups per (b,h) where the device holds n_segs: some CUs with two, some with one.  It is cut
        // into as many pieces as there are segments instead (whole 64-token tiles, at least 256 tokens); a piece that
        // reaches across a segment boundary leaves one local state on either side.
        const int64_t end = (n_segs - 1) * seg_len;
        int64_t piece = seg_len, pieces = n_segs - 1;
        if (d->chunk <= 0) {
            piece = std::max<int64_t>(256, ((end + n_segs - 1) / n_segs + 63) / 64 * 64);
            if (piece >= seg_len) piece = seg_len;
            pieces = (end + piece - 1) / piece;
        }
        p.n_pieces = (int)pieces;
        p.piece_len = (int)piece;
        p.n_slots = (int)(pieces + n_segs);      // at most one more local state per boundary, and the staging slot
    }
    p.off_den = ((size_t)BH * sizeof(int) + 255) / 256 * 256;
    p.off_num = p.off_den + (p.n_segs > 1 ? (size_t)BH * p.n_slots * d->M * sizeof(float) : 0);
    p.total = p.off_num + (p.n_segs > 1 ? (size_t)BH * p.n_slots * d->M * d->D * sizeof(float) : 0);
    return p;
}

void fill_causal_args(flare::CausalArgs& a, const FlareCausalDesc* d)
{
    memset(&a, 0, sizeof(a));
    a.B = d->B; a.H = d->H; a.N = d->N; a.M = d->M; a.D = d->D;
    a.chunk = d->chunk > 0 ? d->chunk : 256;
    a.scale = d->scale;
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = d->q_stride[i]; a.ks[i] = d->k_stride[i]; a.vs[i] = d->v_stride[i]; a.ys[i] = d->y_stride[i];
    }
}

// ---- causal linear --------------------------------------------------------------------
int check_causal_linear_desc(const FlareCausalLinearDesc* d)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->B < 1 || d->H < 1 || d->N < 1 || d->Dk < 1 || d->Dv < 1)
        return fail(FLARE_EINVAL, "B,H,N,Dk,Dv must be >= 1 (got %d,%d,%d,%d,%d)", d->B, d->H, d->N, d->Dk, d->Dv);
    if (d->dtype < FLARE_DT_F32 || d->dtype > FLARE_DT_F16) return fail(FLARE_EINVAL, "unknown dtype %d", d->dtype);
    if (d->Dk > 128 || d->Dv > 128) return fail(FLARE_EUNSUPPORTED, "Dk=%d, Dv=%d: at most 128 supported", d->Dk, d->Dv);
    if (d->n_segs < 0) return fail(FLARE_EINVAL, "n_segs must be >= 0");
    if ((int64_t)d->B * d->H > 65535) return fail(FLARE_EUNSUPPORTED, "B*H must be <= 65535");
    const int64_t* ss[4] = {d->q_stride, d->k_stride, d->v_stride, d->y_stride};
    const int w[4] = {d->Dk, d->Dk, d->Dv, d->Dv};
    const char* nm[4] = {"q", "k", "v", "y"};
    for (int t = 0; t < 4; ++t)
        if (ss[t][2] < w[t]) return fail(FLARE_EINVAL, "%s row stride %lld < row width %d", nm[t], (long long)ss[t][2], w[t]);
    return FLARE_OK;
}

struct CausalLinearPlan { int n_segs, seg_len; size_t total; };

CausalLinearPlan plan_causal_linear(const FlareCausalLinearDesc* d)
{
    const int tile = flare::causal_linear_tile();
    const int64_t BH = (int64_t)d->B * d->H;
    const int64_t tiles = ((int64_t)d->N + tile - 1) / tile;
    // automatic: about four workgroups per compute unit, never more segments than tiles
    int64_t want = d->n_segs > 0 ? d->n_segs : std::max<int64_t>(1, (4 * flare::device_cus() + BH - 1) / BH);
    want = std::min<int64_t>(std::min<int64_t>(want, tiles), 4096);
    const int64_t tiles_per_seg = (tiles + want - 1) / want;
    CausalLinearPlan p;
    p.seg_len = (int)(tiles_per_seg * tile);
    p.n_segs = (int)((tiles + tiles_per_seg - 1) / tiles_per_seg);
    p.total = (size_t)BH * p.n_segs * d->Dk * d->Dv * sizeof(float);
    return p;
}

// ---- triple ---------------------------------------------------------------------------
int check_triple_desc(const FlareTripleDesc* d)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->B < 1 || d->H < 1 || d->N < 1 || d->Dq < 1 || d->Dv < 1)
        return fail(FLARE_EINVAL, "B,H,N,Dq,Dv must be >= 1");
    if (d->dtype < FLARE_DT_F32 || d->dtype > FLARE_DT_F16) return fail(FLARE_EINVAL, "unknown dtype %d", d->dtype);
    if (d->Dq > 64 || d->Dv > 64) return fail(FLARE_EUNSUPPORTED, "Dq=%d, Dv=%d: at most 64 supported", d->Dq, d->Dv);
    if (d->feature_map < 0 || d->feature_map > 1) return fail(FLARE_EINVAL, "feature_map must be 0 or 1");
    if (d->n_splits < 0) return fail(FLARE_EINVAL, "n_splits must be >= 0");
    if (d->H > 65535 || d->B > 65535) return fail(FLARE_EUNSUPPORTED, "B and H must be <= 65535");
    return FLARE_OK;
}

struct TriplePlan { bool mfma; int n_splits, n_parts, tokens_per_split; size_t per_split, off_kk, total; };

bool strides_mult4(const int64_t* s) { return s[0] % 4 == 0 && s[1] % 4 == 0 && s[2] % 4 == 0; }
bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

bool triple_wants_mfma(const FlareTripleDesc* d)
{
    return !(d->flags & FLARE_FLAG_FORCE_GENERIC) && flare::triple_mfma_supported(d->dtype, d->Dq, d->Dv) &&
           strides_mult4(d->q1_stride) && strides_mult4(d->q2_stride) && strides_mult4(d->k1_stride) &&
           strides_mult4(d->k2_stride) && strides_mult4(d->v_stride);
}

TriplePlan plan_triple(const FlareTripleDesc* d)
{
    TriplePlan p;
    p.mfma = triple_wants_mfma(d);
    int s = d->n_splits;
    if (s <= 0) {
        // about two workgroups per compute unit: more splits only add partials to write and merge (the matrix-core
        // state kernel runs one workgroup per split and 16 x 16 x 16 block of the state)
        const int64_t nb = p.mfma ? (int64_t)(d->Dq / 16) * (d->Dv / 16) * (d->Dq / 16) : 1;
        const int64_t per = (int64_t)d->B * d->H * nb;
        s = (int)((2 * flare::device_cus() + per - 1) / per);
        if (s < 1) s = 1;
    }
    int64_t tps = ((int64_t)d->N + s - 1) / s;
    tps = ((tps + 63) / 64) * 64;
    p.tokens_per_split = (int)tps;
    p.n_splits = (int)(((int64_t)d->N + tps - 1) / tps);
    p.n_parts = p.n_splits;
    // sized for whichever kernel family ends up running (misaligned pointers demote to the fp32 kernels)
    p.per_split = flare::triple_partial_floats(d->Dq, d->Dv, false);
    if (p.mfma) p.per_split = std::max(p.per_split, flare::triple_partial_floats(d->Dq, d->Dv, true));
    const size_t bh = (size_t)d->B * d->H;
    p.off_kk = bh * p.n_parts * p.per_split * 4;
    p.off_kk = (p.off_kk + 255) & ~(size_t)255;
    p.total = p.off_kk + bh * d->Dq * d->Dq * 4;
    return p;
}

void fill_triple_args(flare::TripleArgs& a, const FlareTripleDesc* d, const TriplePlan& p)
{
    memset(&a, 0, sizeof(a));
    a.B = d->B; a.H = d->H; a.N = d->N; a.Dq = d->Dq; a.Dv = d->Dv;
    a.feature_map = d->feature_map; a.normalize = d->normalize;
    a.n_splits = p.n_splits; a.tokens_per_split = p.tokens_per_split; a.n_parts = p.n_splits;
    for (int i = 0; i < 3; ++i) {
        a.q1s[i] = d->q1_stride[i]; a.q2s[i] = d->q2_stride[i]; a.k1s[i] = d->k1_stride[i];
        a.k2s[i] = d->k2_stride[i]; a.vs[i] = d->v_stride[i]; a.os[i] = d->o_stride[i];
    }
}

}  // namespace

extern "C" {

int flare_abi_version(void) { return FLARE_ABI_VERSION; }

const char* flare_last_error_string(void) { return g_err; }

const char* flare_mixer_kernel_name(const FlareMixerDesc* desc)
{
    if (check_mixer_desc(desc) != FLARE_OK) return nullptr;
    if (!desc_wants_mfma(desc)) return "generic";
    return desc->dtype == FLARE_DT_BF16 ? "mfma_bf16" : "mfma_f16";
}

int flare_mixer_workspace_bytes(const FlareMixerDesc* desc, size_t* bytes)
{
    if (!bytes) return fail(FLARE_EINVAL, "bytes is NULL");
    int rc = check_mixer_desc(desc);
    if (rc != FLARE_OK) return rc;
    *bytes = mixer_ws_bytes(desc);
    return FLARE_OK;
}

int flare_gather_fwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                     const uint8_t* key_mask, float* z, float* lse, void* workspace,
                     size_t workspace_bytes, void* stream)
{
    int rc = check_mixer_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !z) return fail(FLARE_EINVAL, "q, k, v and z must not be NULL");
    return do_gather(desc, q, k, v, key_mask, z, lse, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int flare_scatter_fwd(const FlareMixerDesc* desc, const void* q, const void* k, const float* z,
                      const uint8_t* key_mask, void* y, void* stream)
{
    int rc = check_mixer_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !z || !y) return fail(FLARE_EINVAL, "q, k, z and y must not be NULL");
    return do_scatter(desc, q, k, z, key_mask, y, static_cast<hipStream_t>(stream));
}

int flare_scatter_fwd_lse(const FlareMixerDesc* desc, const void* q, const void* k, const float* z,
                          const uint8_t* key_mask, void* y, float* lse_tok, void* stream)
{
    int rc = check_mixer_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !z || !y) return fail(FLARE_EINVAL, "q, k, z, y must not be NULL");
    return do_scatter(desc, q, k, z, key_mask, y, static_cast<hipStream_t>(stream), lse_tok);
}

namespace {
struct BwdPlan { int n_splits, tokens_per_split, n_splits0, tokens_per_split0; size_t off_dz, off_dl, off_rm, off_part, total; };

bool bwd_wants_dz32(const FlareMixerDesc* d)
{
    return !(d->flags & FLARE_FLAG_MFMA16) && drop_threshold(d) == 0 && flare::bwd_dz32_supported(d->dtype, d->M, d->D);
}

BwdPlan plan_bwd(const FlareMixerDesc* d)
{
    BwdPlan p;
    const int64_t bh = (int64_t)d->B * d->H;
    const bool f32 = d->dtype == FLARE_DT_F32;      // the fp32 kernels cover 64 latents per workgroup, two workgroups per CU
    const int mblocks = f32 ? (d->M + 63) / 64 : d->M % 256 == 0 ? d->M / 256 : d->M % 128 == 0 ? d->M / 128 : (d->M + 63) / 64;
    // As many workgroups per compute unit over the latent-side grids as the registers of the dq pass allow (two at
    // the larger shapes, see bwd_dq_wgs_per_cu); the dz pass needs fewer and gets three at D = 32 with 64 latents per
    // wave, four below that (measured: 74 -> 66 us at M = 128, D = 16; 203 -> 193 us at M = 128, D = 32), with its
    // own split of the token axis.
    auto split = [&](int per_cu, int& n_splits, int& tokens_per_split) {
        int64_t s = std::max<int64_t>(1, per_cu * flare::device_cus() / (bh * mblocks));
        int64_t tps = ((int64_t)d->N + s - 1) / s;
        tps = (tps + 63) / 64 * 64;
        tokens_per_split = (int)tps;
        n_splits = (int)(((int64_t)d->N + tps - 1) / tps);
    };
    if (bwd_wants_dz32(d)) {
        // the 32x32x16 dz and dq passes: two workgroups per compute unit, ranges a multiple of their four waves' 32-token
        // passes; 256 latents per workgroup in the dz pass, 128 in the dq pass
        auto split32 = [&](int64_t blocks, int& n_splits, int& tokens_per_split) {
            int64_t s = std::max<int64_t>(1, 2 * flare::device_cus() / (bh * blocks));
            int64_t tps = (((int64_t)d->N + s - 1) / s + 127) / 128 * 128;
            if (tps < 512) tps = 512;
            tokens_per_split = (int)tps;
            n_splits = (int)(((int64_t)d->N + tps - 1) / tps);
        };
        split32(mblocks, p.n_splits0, p.tokens_per_split0);
        split32(flare::bwd_dq32_mblocks(d->M), p.n_splits, p.tokens_per_split);
    } else {
        split(f32 ? 2 : flare::bwd_dq_wgs_per_cu(d->D, d->M % 256 == 0 ? 4 : d->M % 128 == 0 ? 2 : 1), p.n_splits, p.tokens_per_split);
        split(f32 ? 2 : d->D <= 16 ? 4 : d->D <= 32 ? (d->M % 256 ? 4 : 3) : 2, p.n_splits0, p.tokens_per_split0);
    }
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    p.off_dz = up((size_t)bh * d->N * 4);
    p.off_dl = p.off_dz + up((size_t)bh * d->M * d->D * 4);
    p.off_rm = p.off_dl + up((size_t)bh * d->M * 4);
    p.off_part = p.off_rm + up((size_t)bh * p.n_splits0 * 4);
    p.total = p.off_part + (size_t)bh * std::max(p.n_splits, p.n_splits0) * d->M * d->D * 4;
    return p;
}

int check_bwd(const FlareMixerDesc* d)
{
    int rc = check_mixer_desc(d);
    if (rc != FLARE_OK) return rc;
    if (d->dtype == FLARE_DT_F32) {
        if (!flare::mixer_bwd_f32_supported(d->M, d->D))
            return fail(FLARE_EUNSUPPORTED, "fp32 mixer backward covers D in {16,32,64}, M %% 16 == 0 (got M=%d, D=%d)", d->M, d->D);
        if (!strides_mult4(d->q_stride) || !strides_mult4(d->k_stride) || !strides_mult4(d->v_stride) || !strides_mult4(d->y_stride))
            return fail(FLARE_EUNSUPPORTED, "fp32 mixer backward needs strides that are multiples of 4 elements");
        return FLARE_OK;
    }
    if (!flare::mixer_bwd_supported(d->dtype, d->M, d->D))
        return fail(FLARE_EUNSUPPORTED, "mixer backward covers bf16/f16, D in {16,32,64}, M %% 32 == 0, M*D <= 65536, and fp32 "
                                        "(got dtype %d, M=%d, D=%d)", d->dtype, d->M, d->D);
    if (!strides_mult8(d->q_stride) || !strides_mult8(d->k_stride) || !strides_mult8(d->v_stride) || !strides_mult8(d->y_stride))
        return fail(FLARE_EUNSUPPORTED, "mixer backward needs strides that are multiples of 8 elements");
    return FLARE_OK;
}
}  // namespace

int flare_mixer_bwd_workspace_bytes(const FlareMixerDesc* desc, size_t* bytes)
{
    if (!bytes) return fail(FLARE_EINVAL, "bytes is NULL");
    int rc = check_bwd(desc);
    if (rc != FLARE_OK) return rc;
    *bytes = plan_bwd(desc).total;
    return FLARE_OK;
}

int flare_mixer_bwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v, const void* y,
                    const float* z, const float* lse_lat, const float* lse_tok, const void* dy,
                    const int64_t dy_stride[3], float* dq, void* dk, void* dv,
                    void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_bwd(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !y || !z || !lse_lat || !lse_tok || !dy || !dy_stride || !dq || !dk || !dv)
        return fail(FLARE_EINVAL, "q, k, v, y, z, lse_lat, lse_tok, dy, dy_stride, dq, dk, dv must not be NULL");
    const bool f32 = desc->dtype == FLARE_DT_F32;
    if (!(f32 ? strides_mult4(dy_stride) : strides_mult8(dy_stride)) || dy_stride[2] < desc->D)
        return fail(FLARE_EINVAL, "dy strides must be multiples of 16 bytes and its rows >= D");
    const void* ptrs[7] = {q, k, v, y, dy, dk, dv};
    for (const void* p : ptrs)
        if (!aligned16(p)) return fail(FLARE_EINVAL, "q, k, v, y, dy, dk, dv must be 16-byte aligned");
    const BwdPlan p = plan_bwd(desc);
    if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    if (workspace_bytes < p.total) return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, p.total);
    if (!aligned16(workspace)) return fail(FLARE_EINVAL, "workspace must be 16-byte aligned");
    flare::MixerBwdArgs a;
    memset(&a, 0, sizeof(a));
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    a.q = q; a.k = k; a.v = v; a.y = y; a.dy = dy; a.z = z; a.lse_lat = lse_lat; a.lse_tok = lse_tok;
    a.delta_tok = reinterpret_cast<float*>(ws);
    a.dz = reinterpret_cast<float*>(ws + p.off_dz);
    a.delta_lat = reinterpret_cast<float*>(ws + p.off_dl);
    a.rho_min = reinterpret_cast<float*>(ws + p.off_rm);
    a.part = reinterpret_cast<float*>(ws + p.off_part);
    a.dq = dq; a.dk = dk; a.dv = dv;
    a.B = desc->B; a.H = desc->H; a.N = desc->N; a.M = desc->M; a.D = desc->D;
    a.n_splits = p.n_splits; a.tokens_per_split = p.tokens_per_split;
    a.n_splits0 = p.n_splits0; a.tokens_per_split0 = p.tokens_per_split0;
    a.no_mfma32 = bwd_wants_dz32(desc) ? 0 : 1;
    a.scale = desc->scale; a.scale_log2 = desc->scale * 1.4426950408889634f;
    a.drop_thr = drop_threshold(desc);
    a.drop_rs = 1.f;
    if (a.drop_thr != 0) {
        a.drop_rs = 1.0f / (1.0f - desc->dropout_p);
        a.seed_lo = (uint32_t)(desc->dropout_seed & 0xffffffffu);
        a.seed_hi = (uint32_t)(desc->dropout_seed >> 32);
    }
    const int64_t nd = (int64_t)desc->N * desc->D;
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = desc->q_stride[i]; a.ks[i] = desc->k_stride[i]; a.vs[i] = desc->v_stride[i];
        a.ys[i] = desc->y_stride[i]; a.dys[i] = dy_stride[i];
    }
    a.dks[0] = a.dvs[0] = (int64_t)desc->H * nd; a.dks[1] = a.dvs[1] = nd; a.dks[2] = a.dvs[2] = desc->D;
    if (desc->flags & FLARE_FLAG_GRAD_LIKE_KV)
        for (int i = 0; i < 3; ++i) { a.dks[i] = desc->k_stride[i]; a.dvs[i] = desc->v_stride[i]; }
    if (f32) return hip_status(flare::launch_mixer_bwd_f32(a, static_cast<hipStream_t>(stream)), "fp32 mixer backward launch");
    return hip_status(flare::launch_mixer_bwd(a, desc->dtype, static_cast<hipStream_t>(stream)), "mixer backward launch");
}

namespace {
// Argument block of the half backwards: the whole-mixer workspace layout, one term of dS switched off (fp32: compiled
// out; bf16 / f16: its softmax weights forced to zero through a log-sum-exp of 1e30, see bwd_half_prep_kernel).
int half_bwd_args(flare::MixerBwdArgs& a, const FlareMixerDesc* desc, void* workspace, size_t workspace_bytes)
{
    int rc = check_bwd(desc);
    if (rc != FLARE_OK) return rc;
    if (desc->dtype != FLARE_DT_F32 && drop_threshold(desc) != 0)
        return fail(FLARE_EUNSUPPORTED, "the bf16 / f16 half backwards do not take attention dropout");
    const BwdPlan p = plan_bwd(desc);
    if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    if (workspace_bytes < p.total) return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, p.total);
    if (!aligned16(workspace)) return fail(FLARE_EINVAL, "workspace must be 16-byte aligned");
    memset(&a, 0, sizeof(a));
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    a.delta_tok = reinterpret_cast<float*>(ws);
    a.dz = reinterpret_cast<float*>(ws + p.off_dz);
    a.delta_lat = reinterpret_cast<float*>(ws + p.off_dl);
    a.rho_min = reinterpret_cast<float*>(ws + p.off_rm);
    a.part = reinterpret_cast<float*>(ws + p.off_part);
    a.B = desc->B; a.H = desc->H; a.N = desc->N; a.M = desc->M; a.D = desc->D;
    a.n_splits = p.n_splits; a.tokens_per_split = p.tokens_per_split;
    a.n_splits0 = p.n_splits0; a.tokens_per_split0 = p.tokens_per_split0;
    a.no_mfma32 = bwd_wants_dz32(desc) ? 0 : 1;
    a.scale = desc->scale; a.scale_log2 = desc->scale * 1.4426950408889634f;
    a.drop_thr = drop_threshold(desc);
    a.drop_rs = 1.f;
    if (a.drop_thr != 0) {
        a.drop_rs = 1.0f / (1.0f - desc->dropout_p);
        a.seed_lo = (uint32_t)(desc->dropout_seed & 0xffffffffu);
        a.seed_hi = (uint32_t)(desc->dropout_seed >> 32);
    }
    const int64_t nd = (int64_t)desc->N * desc->D;
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = desc->q_stride[i]; a.ks[i] = desc->k_stride[i]; a.vs[i] = desc->v_stride[i]; a.ys[i] = desc->y_stride[i];
    }
    a.dks[0] = a.dvs[0] = (int64_t)desc->H * nd; a.dks[1] = a.dvs[1] = nd; a.dks[2] = a.dvs[2] = desc->D;
    if (desc->flags & FLARE_FLAG_GRAD_LIKE_KV)
        for (int i = 0; i < 3; ++i) { a.dks[i] = desc->k_stride[i]; a.dvs[i] = desc->v_stride[i]; }
    return FLARE_OK;
}
}  // namespace

int flare_gather_bwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v, const float* z,
                     const float* lse_lat, const float* dz, float* dq, void* dk, void* dv,
                     void* workspace, size_t workspace_bytes, void* stream)
{
    flare::MixerBwdArgs a;
    int rc = half_bwd_args(a, desc, workspace, workspace_bytes);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !z || !lse_lat || !dz || !dq || !dk || !dv)
        return fail(FLARE_EINVAL, "q, k, v, z, lse_lat, dz, dq, dk, dv must not be NULL");
    const void* ptrs[8] = {q, k, v, z, dz, dq, dk, dv};
    for (const void* p : ptrs)
        if (!aligned16(p)) return fail(FLARE_EINVAL, "q, k, v, z, dz, dq, dk, dv must be 16-byte aligned");
    a.half = 1;
    a.q = q; a.k = k; a.v = v; a.z = z; a.lse_lat = lse_lat;
    a.dz = const_cast<float*>(dz);                 // read only in this mode
    // the scatter term is switched off: its operands only have to be readable
    a.y = v; a.dy = v;
    for (int i = 0; i < 3; ++i) a.ys[i] = a.dys[i] = a.vs[i];
    a.lse_tok = a.delta_tok;
    a.dq = dq; a.dk = dk; a.dv = dv;
    if (desc->dtype != FLARE_DT_F32)
        return hip_status(flare::launch_mixer_bwd(a, desc->dtype, static_cast<hipStream_t>(stream)), "gather backward launch");
    return hip_status(flare::launch_mixer_bwd_f32(a, static_cast<hipStream_t>(stream)), "fp32 gather backward launch");
}

int flare_scatter_bwd(const FlareMixerDesc* desc, const void* q, const void* k, const float* z, const void* y,
                      const float* lse_tok, const void* dy, const int64_t dy_stride[3], float* dq, void* dk, float* dz,
                      void* workspace, size_t workspace_bytes, void* stream)
{
    flare::MixerBwdArgs a;
    int rc = half_bwd_args(a, desc, workspace, workspace_bytes);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !z || !y || !lse_tok || !dy || !dy_stride || !dq || !dk || !dz)
        return fail(FLARE_EINVAL, "q, k, z, y, lse_tok, dy, dy_stride, dq, dk, dz must not be NULL");
    if (!strides_mult4(dy_stride) || dy_stride[2] < desc->D) return fail(FLARE_EINVAL, "dy strides must be multiples of 16 bytes and its rows >= D");
    const void* ptrs[8] = {q, k, z, y, dy, dq, dk, dz};
    for (const void* p : ptrs)
        if (!aligned16(p)) return fail(FLARE_EINVAL, "q, k, z, y, dy, dq, dk, dz must be 16-byte aligned");
    if (desc->dtype != FLARE_DT_F32 && !strides_mult8(dy_stride))
        return fail(FLARE_EINVAL, "dy strides must be multiples of 8 elements");
    a.half = 2;
    a.q = q; a.k = k; a.z = z; a.y = y; a.dy = dy; a.lse_tok = lse_tok;
    for (int i = 0; i < 3; ++i) a.dys[i] = dy_stride[i];
    a.dz = dz;                                     // written by the first pass's merge, read by the other two
    // the gather term is switched off: its operands only have to be readable
    a.v = k;
    for (int i = 0; i < 3; ++i) a.vs[i] = a.ks[i];
    a.lse_lat = a.delta_lat;
    a.dq = dq; a.dk = dk; a.dv = nullptr;
    if (desc->dtype != FLARE_DT_F32)
        return hip_status(flare::launch_mixer_bwd(a, desc->dtype, static_cast<hipStream_t>(stream)), "scatter backward launch");
    return hip_status(flare::launch_mixer_bwd_f32(a, static_cast<hipStream_t>(stream)), "fp32 scatter backward launch");
}

int flare_mixer_fwd(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                    const uint8_t* key_mask, void* y, float* z_out, void* workspace,
                    size_t workspace_bytes, void* stream)
{
    int rc = check_mixer_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !y) return fail(FLARE_EINVAL, "q, k, v and y must not be NULL");
    if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    float* z = z_out;
    if (!z) {
        // z lives at the tail of the workspace; the offset is the same for both plans' maximum
        const size_t need = mixer_ws_bytes(desc);
        if (workspace_bytes < need)
            return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, need);
        const size_t zbytes = (size_t)desc->B * desc->H * desc->M * desc->D * 4;
        z = reinterpret_cast<float*>(static_cast<char*>(workspace) + (need - zbytes));
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    rc = do_gather(desc, q, k, v, key_mask, z, nullptr, workspace, workspace_bytes, st);
    if (rc != FLARE_OK) return rc;
    return do_scatter(desc, q, k, z, key_mask, y, st);
}

namespace {
// Device address of `scratch` on the current device, looked up on the first call there and kept.
int static_scratch(void** out)
{
    constexpr int kMaxDevices = 64;
    static void* ptrs[kMaxDevices] = {};
    static std::mutex mu;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(FLARE_EUNSUPPORTED, "device index %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_status(e, "hipGetSymbolAddress(scratch)");
        if (!p) return fail(FLARE_EHIP, "hipGetSymbolAddress(scratch) returned a null address");
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return FLARE_OK;
}
}  // namespace

int flare_mixer_fwd_dropout(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                            const uint8_t* key_mask, float dropout_p, uint64_t seed, void* y, float* z_out,
                            void* workspace, size_t workspace_bytes, void* stream)
{
    if (!desc) return fail(FLARE_EINVAL, "descriptor is NULL");
    FlareMixerDesc d = *desc;
    d.dropout_p = dropout_p;
    d.dropout_seed = seed;
    return flare_mixer_fwd(&d, q, k, v, key_mask, y, z_out, workspace, workspace_bytes, stream);
}

int flare_mixer_fwd_static(const FlareMixerDesc* desc, const void* q, const void* k, const void* v,
                           const uint8_t* key_mask, void* y, void* stream)
{
    int rc = check_mixer_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !y) return fail(FLARE_EINVAL, "q, k, v and y must not be NULL");
    const size_t need = mixer_ws_bytes(desc);
    if (need > (size_t)FLARE_STATIC_SCRATCH_BYTES)
        return fail(FLARE_EWORKSPACE, "problem needs %zu bytes of scratch, the static buffer holds %zu: use flare_mixer_fwd with a caller-owned workspace",
                    need, (size_t)FLARE_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    rc = static_scratch(&ws);
    if (rc != FLARE_OK) return rc;
    // every partial row and every row of z that is read is written first by this call's own kernels: nothing to clear
    return flare_mixer_fwd(desc, q, k, v, key_mask, y, nullptr, ws, (size_t)FLARE_STATIC_SCRATCH_BYTES, stream);
}

int flare_clock_probe(double milliseconds, int64_t* out, void* stream)
{
    if (!out) return fail(FLARE_EINVAL, "out must not be NULL");
    if (!(milliseconds > 0.0) || milliseconds > 100.0) return fail(FLARE_EINVAL, "milliseconds must be in (0, 100]");
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<long long*>(out), (long long)(milliseconds * 1.0e5));
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? FLARE_OK : fail(FLARE_EHIP, "clock probe launch: %s", hipGetErrorString(e));
}

int flare_causal_workspace_bytes(const FlareCausalDesc* desc, size_t* bytes)
{
    if (!bytes) return fail(FLARE_EINVAL, "bytes is NULL");
    int rc = check_causal_desc(desc);
    if (rc != FLARE_OK) return rc;
    const CausalPlan p = plan_causal(desc);
    *bytes = p.mfma ? p.total : 0;
    return FLARE_OK;
}

namespace {
int causal_run(const FlareCausalDesc* desc, bool decode, const void* q, const void* k, const void* v, void* y,
               float* lse_tok, float* mu, float* den, float* num, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_causal_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !y || !mu || !den || !num)
        return fail(FLARE_EINVAL, "q, k, v, y, mu, den, num must not be NULL");
    flare::CausalArgs a;
    fill_causal_args(a, desc);
    a.q = q; a.k = k; a.v = v; a.y = y; a.mu = mu; a.den = den; a.num = num; a.lse = lse_tok;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (causal_wants_mfma(desc) && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(y)) {
        // matrix-core kernel without a running maximum; it marks the (b,h) it could not validate
        // and the fp32 kernel, launched right behind it, redoes exactly those
        const CausalPlan p = plan_causal(desc);
        if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
        if (workspace_bytes < p.total)
            return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, p.total);
        if (!aligned16(workspace)) return fail(FLARE_EINVAL, "workspace must be 16-byte aligned");
        a.flags = static_cast<int*>(workspace);
        a.n_segs = decode ? 1 : p.n_segs;          // decode steps are sequential by nature
        a.seg_len = decode ? desc->N : p.seg_len;
        a.n_pieces = decode ? 0 : p.n_pieces;
        a.piece_len = decode ? std::max(desc->N, 1) : p.piece_len;
        a.n_slots = decode ? 1 : p.n_slots;
        a.seg_den = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + p.off_den);
        a.seg_num = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + p.off_num);
        hipError_t e = flare::launch_causal_mfma(a, desc->dtype, decode ? 1 : 16, st);
        if (e != hipSuccess) return hip_status(e, "causal (mfma) launch");
        if (decode) return FLARE_OK;      // the decode kernel redoes what it cannot validate itself: one launch
    }
    hipError_t e = decode ? flare::launch_causal_decode(a, desc->dtype, st) : flare::launch_causal_prefill(a, desc->dtype, st);
    return hip_status(e, decode ? "causal decode launch" : "causal prefill launch");
}
}  // namespace

int flare_causal_prefill_fwd(const FlareCausalDesc* desc, const void* q, const void* k, const void* v,
                             void* y, float* mu, float* den, float* num, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return causal_run(desc, false, q, k, v, y, nullptr, mu, den, num, workspace, workspace_bytes, stream);
}

int flare_causal_prefill_fwd_lse(const FlareCausalDesc* desc, const void* q, const void* k, const void* v,
                                 void* y, float* lse_tok, float* mu, float* den, float* num, void* workspace,
                                 size_t workspace_bytes, void* stream)
{
    if (!lse_tok) return fail(FLARE_EINVAL, "lse_tok must not be NULL");
    return causal_run(desc, false, q, k, v, y, lse_tok, mu, den, num, workspace, workspace_bytes, stream);
}

int flare_causal_decode_fwd(const FlareCausalDesc* desc, const void* q, const void* k, const void* v,
                            void* y, float* mu, float* den, float* num, void* workspace,
                            size_t workspace_bytes, void* stream)
{
    return causal_run(desc, true, q, k, v, y, nullptr, mu, den, num, workspace, workspace_bytes, stream);
}

int flare_causal_decode_fwd_lse(const FlareCausalDesc* desc, const void* q, const void* k, const void* v,
                                void* y, float* lse_tok, float* mu, float* den, float* num, void* workspace,
                                size_t workspace_bytes, void* stream)
{
    if (!lse_tok) return fail(FLARE_EINVAL, "lse_tok must not be NULL");
    return causal_run(desc, true, q, k, v, y, lse_tok, mu, den, num, workspace, workspace_bytes, stream);
}

int flare_causal_join(int32_t dtype, int32_t n_groups, int64_t rows, int32_t D, const void* const* y_groups,
                      const float* const* lse_groups, void* y, void* stream)
{
    if (dtype < FLARE_DT_F32 || dtype > FLARE_DT_F16) return fail(FLARE_EINVAL, "unknown dtype %d", dtype);
    if (n_groups < 1 || n_groups > FLARE_JOIN_MAX_GROUPS)
        return fail(FLARE_EINVAL, "n_groups must be in 1..%d (got %d)", FLARE_JOIN_MAX_GROUPS, n_groups);
    if (rows < 0 || D < 1 || D > 128 || D % 8 != 0) return fail(FLARE_EINVAL, "rows must be >= 0, D a multiple of 8 up to 128");
    if (!y_groups || !lse_groups || !y) return fail(FLARE_EINVAL, "y_groups, lse_groups, y must not be NULL");
    flare::CausalJoinArgs a;
    memset(&a, 0, sizeof(a));
    for (int g = 0; g < n_groups; ++g) {
        if (!y_groups[g] || !lse_groups[g]) return fail(FLARE_EINVAL, "group %d has a NULL pointer", g);
        if (!aligned16(y_groups[g])) return fail(FLARE_EINVAL, "group outputs must be 16-byte aligned");
        a.yg[g] = y_groups[g];
        a.lse[g] = lse_groups[g];
    }
    if (!aligned16(y)) return fail(FLARE_EINVAL, "y must be 16-byte aligned");
    a.y = y; a.n_groups = n_groups; a.rows = rows; a.D = D;
    if (rows == 0) return FLARE_OK;
    return hip_status(flare::launch_causal_join(a, dtype, static_cast<hipStream_t>(stream)), "causal join launch");
}

int flare_causal_linear_workspace_bytes(const FlareCausalLinearDesc* desc, size_t* bytes)
{
    if (!bytes) return fail(FLARE_EINVAL, "bytes is NULL");
    int rc = check_causal_linear_desc(desc);
    if (rc != FLARE_OK) return rc;
    *bytes = plan_causal_linear(desc).total;
    return FLARE_OK;
}

int flare_causal_linear_fwd(const FlareCausalLinearDesc* desc, const void* q, const void* k, const void* v,
                            void* y, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_causal_linear_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q || !k || !v || !y) return fail(FLARE_EINVAL, "q, k, v, y must not be NULL");
    const CausalLinearPlan p = plan_causal_linear(desc);
    if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    if (workspace_bytes < p.total)
        return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, p.total);
    if (reinterpret_cast<uintptr_t>(workspace) % 4) return fail(FLARE_EINVAL, "workspace must be 4-byte aligned");
    flare::CausalLinearArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.k = k; a.v = v; a.y = y;
    a.states = static_cast<float*>(workspace);
    a.B = desc->B; a.H = desc->H; a.N = desc->N; a.Dk = desc->Dk; a.Dv = desc->Dv;
    a.n_segs = p.n_segs; a.seg_len = p.seg_len;
    a.inv_n = 1.0f / (float)desc->N;
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = desc->q_stride[i]; a.ks[i] = desc->k_stride[i]; a.vs[i] = desc->v_stride[i]; a.ys[i] = desc->y_stride[i];
    }
    // 16-bit inputs of the sizes the matrix-core kernels take go there when every row is 16-byte aligned
    const bool mfma = !(desc->flags & FLARE_FLAG_FORCE_GENERIC) && flare::causal_linear_mfma_supported(desc->dtype, desc->Dk, desc->Dv) &&
                      strides_mult8(desc->q_stride) && strides_mult8(desc->k_stride) && strides_mult8(desc->v_stride) &&
                      strides_mult8(desc->y_stride) && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(y);
    if (mfma) return hip_status(flare::launch_causal_linear_mfma(a, desc->dtype, static_cast<hipStream_t>(stream)), "causal linear launch");
    return hip_status(flare::launch_causal_linear(a, desc->dtype, static_cast<hipStream_t>(stream)), "causal linear launch");
}

static int mlp_fwd_impl(const FlareMlpDesc* d, int in_dim, int in_act, const float* w_in, const float* b_in, int out_dim,
                        const void* x, const void* w, const float* bias, const float* gamma, const float* beta,
                        const void* res, void* y, void* stream)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->T < 1 || d->L < 1 || d->L > 16) return fail(FLARE_EINVAL, "T >= 1 and 1 <= L <= 16 required (got %lld, %d)", (long long)d->T, d->L);
    if (d->w_dtype != FLARE_DT_BF16 && d->w_dtype != FLARE_DT_F16) return fail(FLARE_EINVAL, "w_dtype must be bf16 or f16");
    const int dts[3] = {d->x_dtype, d->res_dtype, d->y_dtype};
    for (int i = 0; i < 3; ++i)
        if (dts[i] < FLARE_DT_F32 || dts[i] > FLARE_DT_F16) return fail(FLARE_EINVAL, "unknown dtype %d", dts[i]);
    if (d->norm < FLARE_NORM_NONE || d->norm > FLARE_NORM_RMS) return fail(FLARE_EINVAL, "unknown norm %d", d->norm);
    if (d->act < FLARE_ACT_GELU_TANH || d->act > FLARE_ACT_SILU) return fail(FLARE_EINVAL, "unknown activation %d", d->act);
    if (!flare::mlp_mfma_supported(d->w_dtype, d->C)) return fail(FLARE_EUNSUPPORTED, "C=%d: only 32, 64 and 128 are supported", d->C);
    if (!x || !w || !y) return fail(FLARE_EINVAL, "x, w, y must not be NULL");
    if (d->norm != FLARE_NORM_NONE && !gamma) return fail(FLARE_EINVAL, "gamma must not be NULL when a norm is requested");
    if (d->norm != FLARE_NORM_NONE && !(d->eps >= 0.f)) return fail(FLARE_EINVAL, "eps must be >= 0");
    if (in_dim < 0 || in_dim > 4 || out_dim < 0 || out_dim > 4) return fail(FLARE_EINVAL, "in_dim and out_dim must be in [0, 4] (got %d, %d)", in_dim, out_dim);
    const int x_head = 4 * ((d->flags >> 8) & 15), y_head = 4 * ((d->flags >> 12) & 15);
    if ((in_dim || out_dim || x_head || y_head) && (d->flags & FLARE_MLP_EXPAND))
        return fail(FLARE_EINVAL, "FLARE_MLP_EXPAND cannot be combined with in_dim / out_dim / head-padded rows");
    if ((x_head || y_head) && (x_head > 8 || y_head > 8 || in_dim || out_dim))
        return fail(FLARE_EINVAL, "head-padded rows need a head dim of 4 or 8 and cannot be combined with in_dim / out_dim");
    const int64_t x_width = x_head ? 16 * (int64_t)(d->C / x_head) : d->C, y_width = y_head ? 16 * (int64_t)(d->C / y_head) : d->C;
    if (in_dim) {
        if (!w_in || !b_in || !aligned16(w_in) || !aligned16(b_in)) return fail(FLARE_EINVAL, "w_in and b_in must be 16-byte aligned and not NULL when in_dim > 0");
        if (d->norm != FLARE_NORM_NONE) return fail(FLARE_EINVAL, "no norm in front of a lifting first layer");
        if (d->x_stride < in_dim) return fail(FLARE_EINVAL, "x_stride must be >= in_dim");
    } else {
        // every lane moves 4 consecutive elements at a time
        if (d->x_stride < x_width || d->x_stride % 4 || !aligned16(x)) return fail(FLARE_EINVAL, "x: row stride >= the row width, a multiple of 4, base 16-byte aligned");
    }
    if (out_dim) {
        if (res) return fail(FLARE_EINVAL, "res must be NULL when out_dim > 0");
        if (d->y_stride < out_dim) return fail(FLARE_EINVAL, "y_stride must be >= out_dim");
    } else {
        if (d->y_stride < y_width || d->y_stride % 4 || !aligned16(y)) return fail(FLARE_EINVAL, "y: row stride >= the row width, a multiple of 4, base 16-byte aligned");
    }
    if (res && (d->res_stride < d->C || d->res_stride % 4 || !aligned16(res))) return fail(FLARE_EINVAL, "res: row stride >= C, a multiple of 4, base 16-byte aligned");
    if (!aligned16(w) || (bias && !aligned16(bias)) || (gamma && !aligned16(gamma)) || (beta && !aligned16(beta)))
        return fail(FLARE_EINVAL, "w, bias, gamma, beta must be 16-byte aligned");
    flare::MlpArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x; a.res = res; a.y = y; a.w = static_cast<const uint16_t*>(w); a.bias = bias; a.gamma = gamma; a.beta = beta;
    a.T = d->T; a.C = d->C; a.L = d->L;
    a.x_dtype = d->x_dtype; a.res_dtype = d->res_dtype; a.y_dtype = d->y_dtype;
    a.norm = d->norm; a.eps = d->eps; a.act = d->act; a.act_mask = d->act_mask; a.add_mask = d->add_mask;
    a.expand = (d->flags & FLARE_MLP_EXPAND) ? 1 : 0;
    if (a.expand) {
        if (d->L % 2) return fail(FLARE_EINVAL, "FLARE_MLP_EXPAND needs an even number of weight tiles (got L=%d)", d->L);
        a.act_mask = (d->act_mask & 1u) ? 0x55555555u : 0u;      // the activation follows every first product
    }
    a.in_dim = in_dim; a.in_act = in_act ? 1 : 0; a.w_in = w_in; a.b_in = b_in; a.out_dim = out_dim;
    a.x_head = x_head; a.y_head = y_head;
    a.xs = d->x_stride; a.rs = d->res_stride; a.ys = d->y_stride;
    return hip_status(flare::launch_mlp_mfma(a, d->w_dtype, static_cast<hipStream_t>(stream)), "mlp launch");
}

int flare_mlp_fwd(const FlareMlpDesc* d, const void* x, const void* w, const float* bias, const float* gamma,
                  const float* beta, const void* res, void* y, void* stream)
{
    return mlp_fwd_impl(d, 0, 0, nullptr, nullptr, 0, x, w, bias, gamma, beta, res, y, stream);
}

int flare_mlp_io_fwd(const FlareMlpDesc* d, int32_t in_dim, int32_t in_act, const float* w_in, const float* b_in,
                     int32_t out_dim, const void* x, const void* w, const float* bias, const float* gamma,
                     const float* beta, const void* res, void* y, void* stream)
{
    return mlp_fwd_impl(d, in_dim, in_act, w_in, b_in, out_dim, x, w, bias, gamma, beta, res, y, stream);
}

int flare_mlp_bwd_partial_rows(const FlareMlpDesc* d, int32_t* rows)
{
    if (!d || !rows) return fail(FLARE_EINVAL, "descriptor and rows must not be NULL");
    if (d->T < 1) return fail(FLARE_EINVAL, "T >= 1 required");
    *rows = flare::mlp_bwd_partial_rows(d->T);
    return FLARE_OK;
}

// what flare_mlp_bwd and flare_mlp_expand_bwd ask of the descriptor and of the buffers they share
static int check_mlp_bwd_common(const FlareMlpDesc* d, const void* x, const void* dy, const void* w_img, const void* wt_img,
                                const float* bias, const float* gamma, const float* beta, const void* dx, const void* dn,
                                const float* stats, const float* gb_part, const float* gb)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->T < 1 || d->L < 1) return fail(FLARE_EINVAL, "T >= 1 and L >= 1 required (got %lld, %d)", (long long)d->T, d->L);
    if (d->w_dtype != FLARE_DT_BF16 && d->w_dtype != FLARE_DT_F16) return fail(FLARE_EINVAL, "w_dtype must be bf16 or f16");
    if (d->x_dtype < FLARE_DT_F32 || d->x_dtype > FLARE_DT_F16 || d->y_dtype < FLARE_DT_F32 || d->y_dtype > FLARE_DT_F16)
        return fail(FLARE_EINVAL, "unknown dtype");
    if (d->norm < FLARE_NORM_NONE || d->norm > FLARE_NORM_RMS) return fail(FLARE_EINVAL, "unknown norm %d", d->norm);
    if (d->act < FLARE_ACT_GELU_TANH || d->act > FLARE_ACT_SILU) return fail(FLARE_EINVAL, "unknown activation %d", d->act);
    if (!flare::mlp_mfma_supported(d->w_dtype, d->C)) return fail(FLARE_EUNSUPPORTED, "C=%d: only 32, 64 and 128 are supported", d->C);
    if (!x || !dy || !w_img || !wt_img || !dx) return fail(FLARE_EINVAL, "x, dy, w_img, wt_img and dx must not be NULL");
    if (d->norm != FLARE_NORM_NONE && (!gamma || !dn || !stats || !gb_part))
        return fail(FLARE_EINVAL, "gamma, dn, stats and gb_part must not be NULL when a norm is requested");
    if (d->norm != FLARE_NORM_NONE && !(d->eps >= 0.f)) return fail(FLARE_EINVAL, "eps must be >= 0");
    if (d->x_stride < d->C || d->x_stride % 4 || !aligned16(x)) return fail(FLARE_EINVAL, "x: row stride >= C, a multiple of 4, base 16-byte aligned");
    if (d->y_stride < d->C || d->y_stride % 4 || !aligned16(dy)) return fail(FLARE_EINVAL, "dy: row stride (y_stride) >= C, a multiple of 4, base 16-byte aligned");
    const void* ptrs[] = {dx, w_img, wt_img, bias, gamma, beta, dn, stats, gb_part, gb};
    for (const void* p : ptrs)
        if (p && !aligned16(p)) return fail(FLARE_EINVAL, "every buffer must be 16-byte aligned");
    return FLARE_OK;
}

int flare_mlp_bwd(const FlareMlpDesc* d, const void* x, const void* dy, const void* w_img, const void* wt_img,
                  const float* bias, const float* gamma, const float* beta, int32_t add_dy, void* dx, void* a_in,
                  void* g_out, void* dn, float* stats, float* gb_part, float* gb, void* stream)
{
    int rc = check_mlp_bwd_common(d, x, dy, w_img, wt_img, bias, gamma, beta, dx, dn, stats, gb_part, gb);
    if (rc != FLARE_OK) return rc;
    if (d->flags != 0) return fail(FLARE_EUNSUPPORTED, "the backward covers the chain of C x C layers only (flags must be 0)");
    if (d->L > flare::mlp_bwd_max_layers(d->C))
        return fail(FLARE_EUNSUPPORTED, "the backward keeps every layer's slopes in registers: at most %d layers at C=%d (got %d)",
                    flare::mlp_bwd_max_layers(d->C), d->C, d->L);
    if (!a_in || !g_out) return fail(FLARE_EINVAL, "a_in and g_out must not be NULL");
    if (!aligned16(a_in) || !aligned16(g_out)) return fail(FLARE_EINVAL, "every buffer must be 16-byte aligned");
    flare::MlpBwdArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x; a.dy = dy; a.dx = dx;
    a.w = static_cast<const uint16_t*>(w_img); a.wt = static_cast<const uint16_t*>(wt_img);
    a.bias = bias; a.gamma = gamma; a.beta = beta;
    a.a_in = static_cast<uint16_t*>(a_in); a.g_out = static_cast<uint16_t*>(g_out);
    a.dn = static_cast<uint16_t*>(dn); a.stats = stats; a.gb_part = gb_part; a.gb = gb;
    a.T = d->T; a.C = d->C; a.L = d->L;
    a.x_dtype = d->x_dtype; a.dy_dtype = d->y_dtype; a.dx_dtype = d->x_dtype;
    a.norm = d->norm; a.eps = d->eps; a.act = d->act; a.act_mask = d->act_mask; a.add_mask = d->add_mask;
    if (add_dy & ~(FLARE_MLP_BWD_ADD_DY | FLARE_MLP_BWD_ACCUMULATE)) return fail(FLARE_EINVAL, "add_dy holds unknown bits (got %d)", add_dy);
    a.add_dy = add_dy;
    a.xs = d->x_stride; a.dys = d->y_stride; a.dxs = d->C;
    return hip_status(flare::launch_mlp_bwd(a, d->w_dtype, static_cast<hipStream_t>(stream)), "mlp backward launch");
}

int flare_mlp_expand_bwd(const FlareMlpDesc* d, const void* x, const void* dy, const void* w_img, const void* wt_img,
                         const float* bias, const float* gamma, const float* beta, int32_t add_dy, void* dx, void* n_row,
                         void* dy_row, void* h, void* dt, void* dn, float* stats, float* gb_part, float* gb, void* stream)
{
    int rc = check_mlp_bwd_common(d, x, dy, w_img, wt_img, bias, gamma, beta, dx, dn, stats, gb_part, gb);
    if (rc != FLARE_OK) return rc;
    if (d->flags != FLARE_MLP_EXPAND) return fail(FLARE_EINVAL, "flags must be FLARE_MLP_EXPAND");
    if (d->L < 4 || d->L > 16 || (d->L & 1)) return fail(FLARE_EUNSUPPORTED, "L = 2 E tiles with 2 <= E <= 8 (got L = %d)", d->L);
    if (!n_row || !dy_row || !h || !dt) return fail(FLARE_EINVAL, "n_row, dy_row, h and dt must not be NULL");
    if (!aligned16(n_row) || !aligned16(dy_row) || !aligned16(h) || !aligned16(dt)) return fail(FLARE_EINVAL, "every buffer must be 16-byte aligned");
    flare::MlpBwdArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x; a.dy = dy; a.dx = dx;
    a.w = static_cast<const uint16_t*>(w_img); a.wt = static_cast<const uint16_t*>(wt_img);
    a.bias = bias; a.gamma = gamma; a.beta = beta;
    a.a_in = static_cast<uint16_t*>(h); a.g_out = static_cast<uint16_t*>(dt);
    a.n_row = static_cast<uint16_t*>(n_row); a.dy_row = static_cast<uint16_t*>(dy_row);
    a.dn = static_cast<uint16_t*>(dn); a.stats = stats; a.gb_part = gb_part; a.gb = gb;
    a.T = d->T; a.C = d->C; a.L = d->L; a.E = d->L / 2;
    a.x_dtype = d->x_dtype; a.dy_dtype = d->y_dtype; a.dx_dtype = d->x_dtype;
    a.norm = d->norm; a.eps = d->eps; a.act = d->act;
    a.add_dy = add_dy ? 1 : 0;
    a.xs = d->x_stride; a.dys = d->y_stride; a.dxs = d->C;
    return hip_status(flare::launch_mlp_bwd(a, d->w_dtype, static_cast<hipStream_t>(stream)), "mlp expand backward launch");
}

static int check_wgrad_desc(const FlareMlpDesc* d)
{
    if (!d) return fail(FLARE_EINVAL, "descriptor is NULL");
    if (d->T < 1 || d->L < 1) return fail(FLARE_EINVAL, "T >= 1 and L >= 1 required (got %lld, %d)", (long long)d->T, d->L);
    if (d->w_dtype != FLARE_DT_BF16 && d->w_dtype != FLARE_DT_F16) return fail(FLARE_EINVAL, "w_dtype must be bf16 or f16");
    if (!flare::mlp_mfma_supported(d->w_dtype, d->C)) return fail(FLARE_EUNSUPPORTED, "C=%d: only 32, 64 and 128 are supported", d->C);
    if (d->L > 65535) return fail(FLARE_EUNSUPPORTED, "at most 65535 layers");
    return FLARE_OK;
}

int flare_mlp_wgrad_partials(const FlareMlpDesc* d, int32_t* parts)
{
    if (!parts) return fail(FLARE_EINVAL, "parts is NULL");
    int rc = check_wgrad_desc(d);
    if (rc != FLARE_OK) return rc;
    *parts = flare::mlp_wgrad_partials(d->T, d->C, d->L);
    return FLARE_OK;
}

int flare_mlp_wgrad(const FlareMlpDesc* d, const void* a_in, int64_t a_layer_stride, const void* g_out, int64_t g_layer_stride,
                    float* dw_part, float* db_part, float* dw, float* db, void* stream)
{
    int rc = check_wgrad_desc(d);
    if (rc != FLARE_OK) return rc;
    if (!a_in || !g_out || !dw_part) return fail(FLARE_EINVAL, "a_in, g_out and dw_part must not be NULL");
    if (!aligned16(a_in) || !aligned16(g_out) || !aligned16(dw_part) || (db_part && !aligned16(db_part)) ||
        (dw && !aligned16(dw)) || (db && !aligned16(db)))
        return fail(FLARE_EINVAL, "every buffer must be 16-byte aligned");
    if (db && !db_part) return fail(FLARE_EINVAL, "db needs db_part");
    if (a_layer_stride < 0 || g_layer_stride < 0 || a_layer_stride % 8 || g_layer_stride % 8)
        return fail(FLARE_EINVAL, "layer strides must be >= 0 and multiples of 8 elements");
    flare::MlpWgradArgs a;
    memset(&a, 0, sizeof(a));
    a.a_in = static_cast<const uint16_t*>(a_in); a.g_out = static_cast<const uint16_t*>(g_out);
    a.a_lstride = a_layer_stride; a.g_lstride = g_layer_stride;
    a.dw_part = dw_part; a.db_part = db_part; a.dw = dw; a.db = db;
    a.T = d->T; a.C = d->C; a.L = d->L;
    return hip_status(flare::launch_mlp_wgrad(a, d->w_dtype, static_cast<hipStream_t>(stream)), "mlp weight-gradient launch");
}

int flare_triple_workspace_bytes(const FlareTripleDesc* desc, size_t* bytes)
{
    if (!bytes) return fail(FLARE_EINVAL, "bytes is NULL");
    int rc = check_triple_desc(desc);
    if (rc != FLARE_OK) return rc;
    *bytes = plan_triple(desc).total;
    return FLARE_OK;
}

int flare_triple_state_fwd(const FlareTripleDesc* desc, const void* k1, const void* k2, const void* v,
                           float* state, float* kk_state, void* workspace, size_t workspace_bytes,
                           void* stream)
{
    int rc = check_triple_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!k1 || !k2 || !v || !state) return fail(FLARE_EINVAL, "k1, k2, v and state must not be NULL");
    if (desc->normalize && !kk_state) return fail(FLARE_EINVAL, "kk_state is required when normalize != 0");
    if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    const TriplePlan p = plan_triple(desc);
    if (workspace_bytes < p.total)
        return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, p.total);
    flare::TripleArgs a;
    fill_triple_args(a, desc, p);
    a.k1 = k1; a.k2 = k2; a.v = v; a.state = state; a.kk = kk_state;
    a.part = static_cast<float*>(workspace);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool mfma = p.mfma && aligned8(k1) && aligned8(k2) && aligned8(v);
    if (mfma) a.n_parts = p.n_parts;
    a.diag_parts = mfma ? 1 : 0;
    hipError_t e = mfma ? flare::launch_triple_state_mfma(a, desc->dtype, st) : flare::launch_triple_state(a, desc->dtype, st);
    if (e != hipSuccess) return hip_status(e, "triple state launch");
    return hip_status(flare::launch_triple_merge(a, st), "triple merge launch");
}

int flare_triple_out_fwd(const FlareTripleDesc* desc, const void* q1, const void* q2, const float* state,
                         const float* kk_state, void* out, void* stream)
{
    int rc = check_triple_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q1 || !q2 || !state || !out) return fail(FLARE_EINVAL, "q1, q2, state and out must not be NULL");
    if (desc->normalize && !kk_state) return fail(FLARE_EINVAL, "kk_state is required when normalize != 0");
    const TriplePlan p = plan_triple(desc);
    flare::TripleArgs a;
    fill_triple_args(a, desc, p);
    a.q1 = q1; a.q2 = q2; a.out = out; a.state = const_cast<float*>(state); a.kk = const_cast<float*>(kk_state);
    const bool mfma = p.mfma && aligned8(q1) && aligned8(q2) && aligned8(out) && strides_mult4(desc->o_stride);
    hipStream_t st = static_cast<hipStream_t>(stream);
    return hip_status(mfma ? flare::launch_triple_out_mfma(a, desc->dtype, st) : flare::launch_triple_out(a, desc->dtype, st),
                      "triple out launch");
}

int flare_triple_fwd(const FlareTripleDesc* desc, const void* q1, const void* q2, const void* k1,
                     const void* k2, const void* v, float* state, void* out, void* workspace,
                     size_t workspace_bytes, void* stream)
{
    int rc = check_triple_desc(desc);
    if (rc != FLARE_OK) return rc;
    if (!q1 || !q2 || !k1 || !k2 || !v || !state || !out)
        return fail(FLARE_EINVAL, "q1, q2, k1, k2, v, state and out must not be NULL");
    if (!workspace) return fail(FLARE_EWORKSPACE, "workspace is NULL");
    const TriplePlan p = plan_triple(desc);
    if (workspace_bytes < p.total)
        return fail(FLARE_EWORKSPACE, "workspace has %zu bytes, %zu needed", workspace_bytes, p.total);
    float* kk = reinterpret_cast<float*>(static_cast<char*>(workspace) + p.off_kk);
    rc = flare_triple_state_fwd(desc, k1, k2, v, state, kk, workspace, workspace_bytes, stream);
    if (rc != FLARE_OK) return rc;
    return flare_triple_out_fwd(desc, q1, q2, state, kk, out, stream);
}

}  // extern "C"
