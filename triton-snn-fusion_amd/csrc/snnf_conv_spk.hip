// Host side of the convolution + LIF operator on the internal activation layouts (channel-blocked C8, bit-packed BITS):
// argument validation, patch planning and launch of conv_spk_kernel.
#include <algorithm>
#include <array>
#include <cstdio>
#include <map>
#include <mutex>

#include "snnf_conv_spk_kernel.h"

namespace snnf {
namespace {

constexpr int kWaveLds = (static_cast<int>(kMaxLds) - static_cast<int>(kSpkHeaderBytes)) / kSpkWaves / 16 * 16;   // private staging bytes of a wave

struct SpkPlan {
    int PR, PC, PI, RR, RC, region, G, patches_x, patches_y, img_groups;
    double score;
};

// Patch of a wave (PR x PC output pixels of one image, or PI whole planes when a plane has at most 32 pixels) and the
// channel groups per LDS stage G: the patch with the most useful matrix lanes and the smallest halo whose stage fits the
// wave's LDS region and its staging slots; the largest such G (fewer, longer stages).
bool plan_spk(const SpkGeom& g0, int tt, SpkPlan& best, int only_pc = 0, int only_g = 0, bool even = false) {
    best.score = -1.0;
    const int cus = compute_units();
    for (int pc = 1; pc <= 32 && pc <= g0.Wo; ++pc) {
        if (only_pc > 0 && pc != only_pc) continue;
        const int pr = std::min(32 / pc, g0.Ho);
        if (even && ((pc & 1) || (pr & 1))) continue;   // 2x2 windows of the output must lie inside a patch
        const bool whole = pr == g0.Ho && pc == g0.Wo;
        int pi = whole ? std::max(1, std::min(g0.N, 32 / (pr * pc))) : 1;
        // Whole planes of several images per patch: half as many images (idle matrix lanes) when the layer would otherwise have
        // fewer tiles than half the compute units; a tile's K is shared by the eight waves of a workgroup at that size, so tiles
        // are workgroups (512 -> 512 on 2 x 2 planes at batch 64: 64 workgroups of 8 images 24.1 us, 128 of 4 images 21.3 us,
        // 256 of 2 images 22.6 us, single images 34.7 us).
        const int oc_tiles = (g0.Cout + 63) / 64;
        if (pi > 1 && ((g0.N + pi - 1) / pi) * oc_tiles * 2 < cus) pi >>= 1;
        const int rr = (pr - 1) * g0.sh + g0.KH;
        const int rc = (pc - 1) * g0.sw + g0.KW;
        if (rr > 255 || rc > 255) continue;
        const int region = pi * rr * rc;
        int G = 0;
        if (g0.tap_pairs) {
            if (region <= 64 * kSpkSlots && tt * (region + 1) * 16 <= kWaveLds) G = 1;
        } else {
            for (int cand = g0.gpc; cand >= 2; cand >>= 1) {
                if (only_g > 0 && cand > only_g) continue;
                if (cand * region <= 64 * kSpkSlots && tt * (cand * region + 1) * 16 <= kWaveLds) {   // + the dummy item of a timestep
                    G = cand;
                    break;
                }
            }
        }
        if (G == 0) continue;
        const int patches_x = (g0.Wo + pc - 1) / pc;
        const int patches_y = (g0.Ho + pr - 1) / pr;
        const int img_groups = (g0.N + pi - 1) / pi;
        const double lanes = static_cast<double>(img_groups) * patches_x * patches_y * 32.0;
        const double eff = static_cast<double>(g0.N) * g0.Ho * g0.Wo / lanes;
        const double halo = static_cast<double>(region) / (static_cast<double>(pi) * pr * pc);
        // Wide patches store longer runs of a row; stages of 4 slots move in one batch.
        double score = eff / (1.0 + 0.08 * (halo - 1.0)) * (1.0 + 0.004 * std::min(pc, 16));
        if (G * region > 256) score *= 0.97;
        if (score > best.score) best = SpkPlan{pr, pc, pi, rr, rc, region, G, patches_x, patches_y, img_groups, score};
    }
    return best.score > 0.0;
}

// Measured choices for particular layers, registered by the host program (snnf_conv_blocked_tune): patch columns, channel
// groups per stage and waves sharing a tile's K, by layer shape. A choice the kernel cannot run is ignored.
using TunedKey = std::array<int, 13>;
struct TunedPlan { int patch_cols, stage_groups, k_waves; };
std::mutex tuned_mutex;
std::map<TunedKey, TunedPlan>& tuned_plans() {
    static std::map<TunedKey, TunedPlan> plans;
    return plans;
}

bool valid_layout(int layout) { return layout == SNNF_LAYOUT_NCHW || layout == SNNF_LAYOUT_C8 || layout == SNNF_LAYOUT_BITS; }

// A projection shortcut whose sums join the main convolution's accumulators: a pointwise convolution (stride s, no padding)
// of a second bit-packed input with as many output channels and output pixels as the main one.
struct Shortcut {
    const void* const* xs;
    int Cin, H, W, stride_h, stride_w;
    const void* packed_weight;
};

}  // namespace

char* conv_plan_buffer();   // the thread's plan text (snnf_conv_igemm.hip), shared with snnf_conv_last_plan()

namespace {
int conv_lif_blocked_impl(const char* who, const void* const* xs, int x_layout, const void* const* residuals, int res_layout, int T,
                          int N, int Cin, int H, int W, int x_dtype, const void* packed_weight, int Cout, int KH,
                          int KW, int stride_h, int stride_w, int pad_h, int pad_w, const void* v_init, void* out,
                          int out_layout, int64_t out_step_stride, void* v_out, int neuron, float v_threshold,
                          float v_reset, float tau, void* stream, const Shortcut* sc, bool pool2 = false);
}  // namespace

}  // namespace snnf

extern "C" int snnf_conv_blocked_tune(int T, int N, int Cin, int H, int W, int Cout, int KH, int KW, int stride_h, int stride_w,
                                      int pad_h, int pad_w, int shared_frame, int patch_cols, int stage_groups, int k_waves) {
    using namespace snnf;
    if (patch_cols < 0 || patch_cols > 32 || stage_groups < 0 || k_waves < 0 || k_waves > kSpkWaves || (k_waves & (k_waves - 1)) != 0)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_blocked_tune: patch_cols=%d stage_groups=%d k_waves=%d out of range", patch_cols,
                    stage_groups, k_waves);
    const TunedKey key = {T, N, Cin, H, W, Cout, KH, KW, stride_h, stride_w, pad_h, pad_w, shared_frame ? 1 : 0};
    std::lock_guard<std::mutex> lock(tuned_mutex);
    if (patch_cols == 0 && stage_groups == 0 && k_waves == 0) tuned_plans().erase(key);
    else tuned_plans()[key] = TunedPlan{patch_cols, stage_groups, k_waves};
    return SNNF_OK;
}

extern "C" int snnf_conv_lif_blocked(const void* const* xs, int x_layout, const void* const* residuals, int res_layout, int T,
                                     int N, int Cin, int H, int W, int x_dtype, const void* packed_weight, int Cout, int KH,
                                     int KW, int stride_h, int stride_w, int pad_h, int pad_w, const void* v_init, void* out,
                                     int out_layout, int64_t out_step_stride, void* v_out, int neuron, float v_threshold,
                                     float v_reset, float tau, void* stream) {
    return snnf::conv_lif_blocked_impl("snnf_conv_lif_blocked", xs, x_layout, residuals, res_layout, T, N, Cin, H, W, x_dtype, packed_weight,
                                       Cout, KH, KW, stride_h, stride_w, pad_h, pad_w, v_init, out, out_layout, out_step_stride, v_out,
                                       neuron, v_threshold, v_reset, tau, stream, nullptr);
}

extern "C" int snnf_conv_lif_blocked_shortcut(const void* const* xs, const void* const* shortcut_xs, int T, int N, int Cin, int H, int W,
                                              int x_dtype, const void* packed_weight, int Cout, int KH, int KW, int pad_h, int pad_w,
                                              int shortcut_Cin, int shortcut_H, int shortcut_W, int shortcut_stride_h, int shortcut_stride_w,
                                              const void* shortcut_packed_weight, const void* v_init, void* out, int out_layout,
                                              int64_t out_step_stride, void* v_out, int neuron, float v_threshold, float v_reset, float tau,
                                              void* stream) {
    using namespace snnf;
    const char* who = "snnf_conv_lif_blocked_shortcut";
    if (shortcut_xs == nullptr || shortcut_packed_weight == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: shortcut_xs and shortcut_packed_weight must be non-null", who);
    const Shortcut sc = {shortcut_xs, shortcut_Cin, shortcut_H, shortcut_W, shortcut_stride_h, shortcut_stride_w, shortcut_packed_weight};
    return conv_lif_blocked_impl(who, xs, SNNF_LAYOUT_BITS, nullptr, SNNF_LAYOUT_BITS, T, N, Cin, H, W, x_dtype, packed_weight, Cout, KH, KW, 1, 1,
                                 pad_h, pad_w, v_init, out, out_layout, out_step_stride, v_out, neuron, v_threshold, v_reset, tau, stream, &sc);
}

extern "C" int snnf_conv_lif_blocked_avgpool(const void* const* xs, int x_layout, int T, int N, int Cin, int H, int W, int x_dtype,
                                             const void* packed_weight, int Cout, int KH, int KW, int stride_h, int stride_w, int pad_h,
                                             int pad_w, void* out, int64_t out_step_stride, void* v_out, float v_threshold, float v_reset,
                                             float tau, void* stream) {
    return snnf::conv_lif_blocked_impl("snnf_conv_lif_blocked_avgpool", xs, x_layout, nullptr, 0, T, N, Cin, H, W, x_dtype, packed_weight, Cout, KH,
                                       KW, stride_h, stride_w, pad_h, pad_w, nullptr, out, SNNF_LAYOUT_C8, out_step_stride, v_out, 1, v_threshold,
                                       v_reset, tau, stream, nullptr, true);
}

namespace snnf {
namespace {
int conv_lif_blocked_impl(const char* who, const void* const* xs, int x_layout, const void* const* residuals, int res_layout, int T,
                          int N, int Cin, int H, int W, int x_dtype, const void* packed_weight, int Cout, int KH,
                          int KW, int stride_h, int stride_w, int pad_h, int pad_w, const void* v_init, void* out,
                          int out_layout, int64_t out_step_stride, void* v_out, int neuron, float v_threshold,
                          float v_reset, float tau, void* stream, const Shortcut* sc, bool pool2) {
    if (xs == nullptr || packed_weight == nullptr || out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: xs, packed_weight and out must be non-null", who);
    if (T < 1 || N < 1 || Cin < 1 || H < 1 || W < 1 || Cout < 1 || KH < 1 || KW < 1 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: bad extent (T=%d N=%d Cin=%d H=%d W=%d Cout=%d K=%dx%d s=%dx%d p=%dx%d)", who,
                    T, N, Cin, H, W, Cout, KH, KW, stride_h, stride_w, pad_h, pad_w);
    if (T > SNNF_MAX_T_PER_LAUNCH)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_temporal_length: T=%d exceeds %d", who, T, SNNF_MAX_T_PER_LAUNCH);
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_dtype: the internal layouts hold bf16 or fp16 activations", who);
    if (x_layout != SNNF_LAYOUT_C8 && x_layout != SNNF_LAYOUT_BITS && x_layout != SNNF_LAYOUT_NCHW)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_layout: inputs must be in C8 or BITS layout (or one dense frame of at most 8 channels)", who);
    if (!valid_layout(out_layout) || (residuals != nullptr && !valid_layout(res_layout)))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: unknown layout code", who);
    if (!neuron && out_layout == SNNF_LAYOUT_BITS)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_layout: an output without a neuron cannot be bit-packed", who);
    if (neuron && !(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_tau: tau must be nonzero", who);
    if (H + 2 * pad_h < KH || W + 2 * pad_w < KW)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_kernel: kernel larger than padded input", who);
    if (2 * pad_h > KH || 2 * pad_w > KW)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_padding: padding %dx%d too large for kernel %dx%d", who, pad_h, pad_w, KH, KW);
    // Bytes a tensor in a layout is accessed by: bit-packed tensors by single bytes, blocked inputs by 16-byte groups, blocked
    // outputs and residuals by 4 channels (8 bytes), dense tensors by elements.
    auto need_align = [](int layout, bool as_input) -> size_t { return layout == SNNF_LAYOUT_BITS ? 1 : (layout == SNNF_LAYOUT_C8 ? (as_input ? 16 : 8) : 2); };
    if (!aligned_to(packed_weight, 16) || !aligned_to(out, need_align(out_layout, false)) || (out_step_stride % need_align(out_layout, false)) != 0 ||
        (v_init != nullptr && !aligned_to(v_init, 4)) || (v_out != nullptr && !aligned_to(v_out, 4)))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: packed_weight, out (and its step stride) or a membrane pointer is misaligned", who);
    bool shared = T > 1;
    for (int t = 0; t < T; ++t) {
        if (xs[t] == nullptr || !aligned_to(xs[t], need_align(x_layout, true)))
            return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: xs[%d] is null or misaligned for its layout", who, t);
        if (residuals != nullptr && (residuals[t] == nullptr || !aligned_to(residuals[t], need_align(res_layout, false))))
            return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: residuals[%d] is null or misaligned for its layout", who, t);
        shared = shared && xs[t] == xs[0];
    }
    if (x_layout == SNNF_LAYOUT_NCHW && (!shared || Cin > 8))
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_layout: a dense input must be one frame of at most 8 channels shared by all timesteps (Cin=%d)", who, Cin);
    if (sc != nullptr) {
        // The shortcut's sums are K steps of the main tile: same output pixels (a main convolution that keeps the plane, the
        // shortcut's stride taking its own input down to it), whole pairs of channel groups, bit-packed input like the main one.
        if (sc->Cin < 1 || sc->H < 1 || sc->W < 1 || sc->stride_h < 1 || sc->stride_w < 1)
            return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: bad shortcut extent (Cin=%d H=%d W=%d s=%dx%d)", who, sc->Cin, sc->H, sc->W, sc->stride_h, sc->stride_w);
        if (KH != 2 * pad_h + 1 || KW != 2 * pad_w + 1 || (sc->H - 1) / sc->stride_h + 1 != H || (sc->W - 1) / sc->stride_w + 1 != W)
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shortcut: the main convolution must keep its %dx%d plane and the shortcut (%dx%d, stride %dx%d) must land on it",
                        who, H, W, sc->H, sc->W, sc->stride_h, sc->stride_w);
        if (sc->Cin % 16 != 0 || Cin % 16 != 0 || shared || T < 3)
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shortcut: needs channel counts that are multiples of 16, at least 3 timesteps and an input per timestep", who);
        if (!aligned_to(sc->packed_weight, 16))
            return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: shortcut_packed_weight is misaligned", who);
        if (static_cast<int64_t>(N) * (sc->Cin / 8) * sc->H * sc->W >= (1LL << 27))
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: shortcut input too large for 32-bit offsets", who);
        for (int t = 0; t < T; ++t)
            if (sc->xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: shortcut_xs[%d] is null", who, t);
    }

    SpkGeom g = {};
    g.N = N; g.Cin = Cin; g.H = H; g.W = W; g.Cout = Cout; g.KH = KH; g.KW = KW;
    g.sh = stride_h; g.sw = stride_w; g.ph = pad_h; g.pw = pad_w;
    g.Ho = (H + 2 * pad_h - KH) / stride_h + 1;
    g.Wo = (W + 2 * pad_w - KW) / stride_w + 1;
    g.C8in = (Cin + 7) / 8;
    g.C8out = (Cout + 7) / 8;
    const int64_t in_items = static_cast<int64_t>(N) * g.C8in * H * W;
    const int64_t out_elems = static_cast<int64_t>(N) * g.C8out * 8 * g.Ho * g.Wo;
    if (in_items >= (1LL << 27) || out_elems >= (1LL << 30) || static_cast<int64_t>(T) * N * g.C8out * g.Ho * g.Wo >= (1LL << 31))
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: tensor too large for 32-bit offsets", who);
    if (out_layout == SNNF_LAYOUT_BITS && (out_step_stride < 0 || out_step_stride >= (1LL << 31) / T))
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: bit-packed output beyond 2 GiB", who);
    const PackGeom pg = make_pack_geom(Cout, Cin, KH, KW, false);
    g.gpc = pg.CK / 8;
    g.npairs = pg.npairs;
    g.nocf = pg.nocf;
    g.tap_pairs = pg.CK == 8 ? 1 : 0;
    g.taps = KH * KW;
    g.frag_stride = static_cast<int64_t>(pg.nchunks) * pg.npairs * (kFragBytes / 2);
    g.T = T;
    g.shared_x = shared ? 1 : 0;
    g.in_layout = x_layout;
    g.res_layout = residuals != nullptr ? res_layout : -1;
    g.out_layout = out_layout;
    g.analog_out = neuron ? 0 : 1;
    g.out_step_stride = out_step_stride;

    // Timesteps side by side: 4 (2 for T == 2, 1 for a single step or a shared frame), fewer when the halo does not fit.
    int tt = shared || T == 1 ? 1 : (T == 2 ? 2 : 4);
    TunedPlan tuned = {0, 0, 0};
    {
        const TunedKey key = {T, N, Cin, H, W, Cout, KH, KW, stride_h, stride_w, pad_h, pad_w, shared ? 1 : 0};
        std::lock_guard<std::mutex> lock(tuned_mutex);
        const auto it = tuned_plans().find(key);
        if (it != tuned_plans().end()) tuned = it->second;
    }
    SpkPlan pl = {};
    if (pool2 && (!neuron || T != 4 || (g.Ho & 1) || (g.Wo & 1) || residuals != nullptr || v_init != nullptr || Cout % 8 != 0))
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_pool: needs four timesteps, a neuron from the zero membrane, no residual, an even %dx%d output plane and whole channel groups",
                    who, g.Ho, g.Wo);
    bool planned = (tuned.patch_cols > 0 || tuned.stage_groups > 0) && plan_spk(g, tt, pl, tuned.patch_cols, tuned.stage_groups, pool2);
    const bool tuned_patch = planned;
    for (; !planned && tt >= 1; tt >>= 1) {
        planned = plan_spk(g, tt, pl, 0, 0, pool2);
        if (planned) break;
        if (pool2) break;   // the pooled store covers the four steps of one window
    }
    if (!planned)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: no patch of this layer fits a wave's LDS region (kernel %dx%d, stride %dx%d)",
                    who, KH, KW, stride_h, stride_w);
    const int windows = shared ? 1 : (T + tt - 1) / tt;
    if (neuron && windows > 1 && v_out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: v_out is required when the timesteps take %d windows of %d (it carries the membrane between them)",
                    who, windows, tt);
    g.PR = pl.PR; g.PC = pl.PC; g.PI = pl.PI; g.RR = pl.RR; g.RC = pl.RC; g.region = pl.region; g.G = pl.G;
    g.patches_x = pl.patches_x;
    g.patches_img = pl.patches_x * pl.patches_y;
    g.n_patches = pl.img_groups * g.patches_img;
    g.nstages = (g.C8in + g.G - 1) / g.G;
    g.IT = g.G * g.region;
    g.JT = (g.IT + 63) / 64;
    g.lds_wave_bytes = tt * (g.IT + 1) * 16;
    const int oc_tiles = (Cout + 63) / 64;
    g.n_items = g.n_patches * oc_tiles;
    // Split K over waves of a workgroup while the layer has fewer items than the machine has SIMDs (one wave each) and
    // every wave still gets at least one stage.
    const int cus = compute_units();
    int wk_log2 = 0;
    while (wk_log2 < 3 && static_cast<int64_t>(g.n_items) << wk_log2 < static_cast<int64_t>(cus) * 6 && g.nstages >= (2 << wk_log2)) ++wk_log2;
    bool tuned_split = false;
    if (tuned.k_waves > 0) {
        int want = 0;
        while ((1 << want) < tuned.k_waves) ++want;
        if (g.nstages >= (1 << want)) {
            wk_log2 = want;
            tuned_split = true;
        }
    }
    g.wk_log2 = wk_log2;
    const int tiles_per_block = kSpkWaves >> wk_log2;
    // Workgroups that are resident together: one per compute unit, or two where a wave needs at most a quarter of a SIMD's
    // registers (one timestep's accumulators) and two staging areas fit the LDS. The tiles are dealt evenly over as many
    // rounds as that takes.
    const size_t lds_bytes = std::max(kSpkHeaderBytes + static_cast<size_t>(kSpkWaves) * g.lds_wave_bytes, wk_log2 > 0 ? kSpkHeaderBytes + kSpkPartialBytes : size_t{0});
    const int resident = cus * ((tt == 1 && 2 * (lds_bytes + 1024) <= kMaxLds) ? 2 : 1);
    const int blocks = (g.n_items + tiles_per_block - 1) / tiles_per_block;
    g.iters = (blocks + resident - 1) / resident;
    const int grid = (blocks + g.iters - 1) / g.iters;
    g.d_ppx = make_fast_div(g.PR * g.PC);
    g.d_PC = make_fast_div(g.PC);
    g.d_region = make_fast_div(g.region);
    g.d_rrrc = make_fast_div(g.RR * g.RC);
    g.d_RC = make_fast_div(g.RC);
    g.d_n_patches = make_fast_div(g.n_patches);
    g.d_patches_img = make_fast_div(g.patches_img);
    g.d_patches_x = make_fast_div(g.patches_x);
    g.d_gpc = make_fast_div(g.gpc);
    const int hg = g.tap_pairs ? 1 : g.G / 2;
    const int nst = g.tap_pairs ? g.npairs : g.taps * hg;
    g.kw_mul = (KW & (KW - 1)) == 0 ? 65536 / KW : 65536 / KW + 1;
    for (int tap = 0; tap < KH * KW; ++tap)
        if (((tap * g.kw_mul) >> 16) != tap / KW)
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_kernel: kernel %dx%d too large", who, KH, KW);
    g.gpc_log2 = 0;
    while ((1 << g.gpc_log2) < g.gpc) ++g.gpc_log2;
    g.hg_log2 = 0;
    while ((1 << g.hg_log2) < hg) ++g.hg_log2;
    g.pair_tap_stride = g.tap_pairs ? 1 : g.gpc / 2;
    if (nst > kSpkMaxSteps)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_kernel: %d matrix steps per stage exceed %d (kernel %dx%d)", who, nst, kSpkMaxSteps, KH, KW);
    PackGeom pg2 = {};
    if (sc != nullptr) {
        pg2 = make_pack_geom(Cout, sc->Cin, 1, 1, false);
        const int gpc2 = pg2.CK / 8;
        if (tt != 4 || g.tap_pairs || gpc2 % g.G != 0 || nst + 4 + hg + 4 > kSpkMaxSteps + 4)
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shortcut: this layer's plan (window %d, %d channel groups per stage, %d steps) has no room for a shortcut",
                        who, tt, g.G, nst);
        g.sc_C8 = sc->Cin / 8;
        g.sc_stages = (g.sc_C8 + g.G - 1) / g.G;
        g.sc_H = sc->H; g.sc_W = sc->W; g.sc_sh = sc->stride_h; g.sc_sw = sc->stride_w;
        g.sc_gpc_log2 = 0;
        while ((1 << g.sc_gpc_log2) < gpc2) ++g.sc_gpc_log2;
        g.sc_npairs = pg2.npairs;
        g.sc_frag_stride = static_cast<int64_t>(pg2.nchunks) * pg2.npairs * (kFragBytes / 2);
    }
    g.d_hg = make_fast_div(hg);
    g.d_nst = make_fast_div(nst);
    g.d_KW = make_fast_div(KW);

    SpkLaunch L = {};
    for (int t = 0; t < T; ++t) {
        L.xs.p[t] = xs[t];
        if (residuals != nullptr) L.residuals.p[t] = residuals[t];
        if (sc != nullptr) L.residuals.p[t] = sc->xs[t];   // the second input travels in the residual's place (a shortcut launch has no residual)
    }
    if (sc != nullptr) {
        L.wpacked2 = static_cast<const uint16_t*>(sc->packed_weight);
        L.bias2 = reinterpret_cast<const float*>(L.wpacked2 + packed_weight_elems(pg2));
    }
    L.g = g;
    L.wpacked = static_cast<const uint16_t*>(packed_weight);
    L.bias = reinterpret_cast<const float*>(L.wpacked + packed_weight_elems(pg));
    L.v_init = neuron ? static_cast<const float*>(v_init) : nullptr;
    L.out = out;
    L.v_out = neuron ? static_cast<float*>(v_out) : nullptr;
    L.lif = make_lif_params(v_threshold, v_reset, tau);
    L.grid = grid;
    L.lds_bytes = lds_bytes;
    L.stream = as_stream(stream);
    const bool fast_epi = neuron && (out_layout == SNNF_LAYOUT_BITS || pool2) && (residuals == nullptr || res_layout == SNNF_LAYOUT_BITS) &&
                          L.lif.charge_mode == CHARGE_SCALE && L.lif.inv_tau == 0.5f && L.lif.v_reset == 0.0f &&
                          L.lif.v_threshold >= 1e-30f && L.lif.v_threshold <= 1e30f &&   // its multiples by 2^t stay normal numbers
                          v_init == nullptr && windows == 1 && Cout % 8 == 0;
    snprintf(snnf::conv_plan_buffer(), 256,
             "kernel=blocked variant=%d window=%d launches=1 tile=%dx%dx%d halo=%dx%d waves=8x1x%d oc_tiles=%d px_tiles=%d "
             "stage_chunks=%d run=0 lds=%zu grid=%d tuned=%d shortcut_stages=%d",
             (wk_log2 > 0 ? 50 : 40) + tt + (fast_epi ? 20 : 0), shared ? T : tt, g.PI, g.PR, g.PC, g.RR, g.RC, 1 << wk_log2, oc_tiles, g.n_patches, g.G,
             L.lds_bytes, grid, (tuned_patch ? 1 : 0) + (tuned_split ? 2 : 0), g.sc_stages);
    L.fast_epilogue = fast_epi;
    if (pool2) {
        if (!fast_epi || windows != 1 || (tt != 4 && !shared))
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_pool: the pooled output needs the usual neuron (tau 2, hard reset to 0) and the four steps in one window", who);
        L.g.pool2 = 1;
        if (x_layout == SNNF_LAYOUT_NCHW) return x_dtype == SNNF_BF16 ? launch_conv_spk_bf16_frame(L, true) : launch_conv_spk_f16_frame(L, true);
        return x_dtype == SNNF_BF16 ? launch_conv_spk_bf16_pooled(L, tt) : launch_conv_spk_f16_pooled(L, tt);
    }
    if (sc != nullptr) return x_dtype == SNNF_BF16 ? launch_conv_spk_bf16_shortcut(L) : launch_conv_spk_f16_shortcut(L);
    if (x_layout == SNNF_LAYOUT_NCHW) return x_dtype == SNNF_BF16 ? launch_conv_spk_bf16_frame(L, false) : launch_conv_spk_f16_frame(L, false);
    if (x_layout == SNNF_LAYOUT_BITS) return x_dtype == SNNF_BF16 ? launch_conv_spk_bf16_bits(L, tt) : launch_conv_spk_f16_bits(L, tt);
    return x_dtype == SNNF_BF16 ? launch_conv_spk_bf16_c8(L, tt) : launch_conv_spk_f16_c8(L, tt);
}

}  // namespace
}  // namespace snnf
