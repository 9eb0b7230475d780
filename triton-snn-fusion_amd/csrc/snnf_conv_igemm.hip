// Host side of the implicit-GEMM conv+LIF operator: argument validation, tile planning and launch.
#include <algorithm>
#include <cstdio>
#include "snnf_conv_common.h"

#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>

namespace snnf {
namespace {

// Largest number of distinct input rows (global id n * H + ih) any tile row-band touches.
int max_tile_rows(const ConvGeom& g) {
    const int total_rows = g.N * g.Ho;
    if (g.Ho % g.TH == 0) return (g.TH - 1) * g.sh + g.KH;  // no band straddles two images
    int worst = 0;
    for (int ty = 0; ty < g.tiles_y; ++ty) {
        const int q0 = ty * g.TH;
        const int q1 = (q0 + g.TH < total_rows ? q0 + g.TH : total_rows) - 1;
        const int n0 = q0 / g.Ho, n1 = q1 / g.Ho;
        const int lo = n0 * g.H + (q0 - n0 * g.Ho) * g.sh - g.ph;
        const int hi = n1 * g.H + (q1 - n1 * g.Ho) * g.sh - g.ph + g.KH - 1;
        if (hi - lo + 1 > worst) worst = hi - lo + 1;
    }
    return worst;
}

struct Plan {
    int TH, TW, tiles_x, tiles_y, NR, WT, wm_log2, wn_log2, oc_tiles;
    size_t lds_bytes;
};

// Picks the wave arrangement (WM x WN) and the output tile (TH rows of the flattened (n, oh) space x TW columns,
// TH * TW <= WM * 64) that keep the most matrix lanes and CUs busy, under the LDS and staging-slot limits.
bool plan_uncached(const ConvGeom& g0, int t_in, int tt, int load_mode, bool want_vec8, Plan& best_plan) {
    // tt == 0: time-outer kernel (one timestep in LDS, two workgroups per CU, its own staging depth and LDS stage).
    const bool pair_shift = load_mode == LOAD_PAIR32;
    const int rows = g0.N * g0.Ho;
    const int groups = 1 << g0.groups_log2;
    const int max_spatial_items = tt == 0 ? kConvThreads * (load_mode == LOAD_PAIR32 ? 4 : 2)
                                           : kConvThreads * (staging_items(load_mode) / tt);
    const int cus = compute_units() * (tt == 0 ? 2 : 1);
    double best = -1.0;
    // Tiles normally fill the waves' pixel lanes (TH * TW == PT where the layer allows). When no such tile fits the staging
    // slots or LDS (large kernels at stride 2 on channel counts off the fast paths), tiles of half, a quarter, ... of the
    // lanes are tried: idle lanes, but the layer runs.
    for (int shrink = 1; shrink <= 16 && best <= 0.0; shrink *= 2)
    for (int wn_log2 = 0; wn_log2 <= 2; ++wn_log2) {
        const int wm_log2 = 2 - wn_log2;
        const int PT = (1 << wm_log2) * 32 * kNPF;
        const int OT = (1 << wn_log2) * 32 * (tt == 0 ? 1 : kNOF);   // the time-outer kernel gives a wave 32 channels
        const int oc_tiles = (g0.Cout + OT - 1) / OT;
        const double oc_eff = static_cast<double>(g0.Cout) / (static_cast<double>(oc_tiles) * OT);
        for (int tw = 1; tw <= g0.Wo && tw <= PT; ++tw) {
            int th = PT / tw / shrink;
            if (th < 1) continue;
            if (th > rows) th = rows;
            ConvGeom c = g0;
            c.TW = tw;
            c.TH = th;
            c.tiles_x = (g0.Wo + tw - 1) / tw;
            c.tiles_y = (rows + th - 1) / th;
            c.NR = max_tile_rows(c);
            c.WT = (tw - 1) * g0.sw + g0.KW + (pair_shift ? 1 : 0);
            c.WT = (c.WT + 1) & ~1;
            size_t bytes = static_cast<size_t>(t_in) * c.NR * c.WT * c.pitch;
            if (tt == 0) {
                bytes += c.pitch + kToutStageBytes;                      // zero pixel + per-wave epilogue stage
                if (bytes * 2 > kMaxLds) continue;                      // two workgroups per CU
            } else {
                if (bytes < kEpiBytes) bytes = kEpiBytes;
                bytes += c.pitch;
                if (bytes > kMaxLds) continue;
            }
            if (groups * c.NR * (c.WT / 2) > max_spatial_items) continue;
            const double work = static_cast<double>(c.tiles_x) * c.tiles_y * oc_tiles;
            const double lane_eff = static_cast<double>(rows) * g0.Wo / (static_cast<double>(c.tiles_x) * c.tiles_y * PT);
            const double waves = work < cus ? 1.0 : static_cast<double>(static_cast<long long>((work + cus - 1) / cus));
            const double fill = work / (waves * cus);
            const double halo = static_cast<double>(c.NR) * c.WT / (static_cast<double>(th) * tw);
            double score = lane_eff * oc_eff * fill / (1.0 + 0.05 * (halo - 1.0)) / (1.0 + 0.1 * (oc_tiles - 1));
            // 16-byte stores need runs of 8 contiguous output pixels: full-width rows or tile widths that are multiples of 8.
            const bool runs = want_vec8 && ((tw == g0.Wo && (g0.Wo % 8 == 0 || g0.Ho == 1)) || tw % 8 == 0);
            if (!runs) score *= 0.6;
            if (score > best) {
                best = score;
                best_plan = Plan{th, tw, c.tiles_x, c.tiles_y, c.NR, c.WT, wm_log2, wn_log2, oc_tiles, bytes};
            }
        }
    }
    return best > 0.0;
}

// Tile plan of the 8-wave matrix kernel: wave arrangement WM x WN (WM * WN == 8; a wave owns 32 pixels x 64 channels)
// and an output tile of TH x TW pixels inside one image (TH * TW <= WM * 32). `fast`: every tile is full and runs of 8
// tile pixels are contiguous, 16-byte aligned runs in memory.
struct MmPlan {
    int TH, TW, tiles_x, tiles_y, NR, WT, wm_log2, wn_log2, wk_log2, oc_tiles, run, all_full, stage_off, stage_chunks, pitch;
    size_t lds_bytes;
    int nw;          // waves per workgroup: 8 (one workgroup per CU) or 4 (two)
    double score;
    int TI;          // images per tile: > 1 only for tiles that are whole output planes (small planes, deep stages)
};

// `vec`: widest aligned spike access the operands allow (8 or 4 elements, 0 = none). The WK waves that split K of one
// tile cost an LDS reduction, so K is only split when the unsplit tiling leaves most of the machine idle.
bool plan_mm_uncached(const ConvGeom& g0, int tt, int load_mode, int vec, int nw, MmPlan& best_plan) {
    const bool pair_shift = load_mode == LOAD_PAIR32;
    const int groups = 1 << g0.groups_log2;
    const int slots = (load_mode == LOAD_PAIR32 ? 8 : 4) / tt;           // staging items per thread (mm_staging_slots)
    const int nw_log2 = nw == 8 ? 3 : 2;
    const int cus = compute_units() * (8 / nw);                  // workgroup slots of the machine
    const size_t lds_cap = kMaxLds * nw / 8;                      // per workgroup
    const size_t stage_bytes = nw * kMmStageBytesPerWave + kMmBiasBytes;   // epilogue stages + the workgroup's bias values
    double best = -1.0;
    for (int wk_log2 = 0; wk_log2 <= nw_log2; ++wk_log2) {
        if ((1 << wk_log2) > g0.npairs) break;
        // Measured on layers that fill the machine without it: splitting pays from K of about 1152 on. A layer of real size
        // (2^18 outputs per timestep or more) whose unsplit tiles occupy less than a quarter of the CUs splits at any K
        // (with the bar at a half, the 3x3/2 and 1x1/2 64->128 layers at 56x56 lost 25-35 %).
        const double outputs = static_cast<double>(g0.N) * g0.Ho * g0.Wo * g0.Cout;
        const double unsplit_groups = outputs / (nw * 64.0 * 32.0);
        const bool starved = outputs >= 262144.0 && unsplit_groups * 4.0 < cus;
        if (wk_log2 > 0 && g0.nchunks * g0.npairs < 72 && !starved) break;
        const int max_items = nw * 64 * ((wk_log2 > 0 && load_mode == LOAD_PAIR32 && tt >= 2) ? slots / 2 : slots);
        for (int wn_log2 = 0; wn_log2 + wk_log2 <= nw_log2; ++wn_log2) {
            const int wm_log2 = nw_log2 - wn_log2 - wk_log2;
            const int PT = (1 << wm_log2) * 32;
            const int OT = (1 << wn_log2) * 64;
            const int oc_tiles = (g0.Cout + OT - 1) / OT;
            const double oc_eff = static_cast<double>(g0.Cout) / (static_cast<double>(oc_tiles) * OT);
            for (int tw = 1; tw <= g0.Wo && tw <= PT; ++tw) {
                int th = PT / tw;
                if (th > g0.Ho) th = g0.Ho;
                const int tiles_x = (g0.Wo + tw - 1) / tw;
                const int tiles_y = (g0.Ho + th - 1) / th;
                const int NR = (th - 1) * g0.sh + g0.KH;
                int WT = (tw - 1) * g0.sw + g0.KW + (pair_shift ? 1 : 0);
                WT = (WT + 1) & ~1;
                // A tile that is a whole output plane may take several images (stacked halo tiles): small planes then
                // still fill the 32-pixel waves.
                const int ti_max = (th == g0.Ho && tw == g0.Wo) ? std::max(1, std::min(g0.N, PT / (th * tw))) : 1;
              for (int ti = 1; ti <= ti_max; ++ti) {
                const int NRT = ti * NR;                           // stacked halo rows
                const int img_groups = (g0.N + ti - 1) / ti;
                // An LDS stage holds as many packed channel chunks as fit (fewer barriers and exposed load latencies per tile).
                // fp32 tensors: a stage holds real chunks, each pixel's channels twice (high and low bf16 terms side by side).
                const int row_mult = g0.nchunks != g0.nchunks_r ? 2 : 1;
                int sc = 1;
                while (sc * 2 <= g0.nchunks_r && sc * 2 * g0.CK * row_mult <= 256 &&
                       static_cast<size_t>(tt) * NRT * WT * (sc * 2 * g0.CK * 2 * row_mult + 16) + stage_bytes <= lds_cap &&
                       sc * 2 * groups * NRT * (WT / 2) <= max_items)
                    sc *= 2;
                const int pitch = sc * g0.CK * 2 * row_mult + 16;
                size_t tiles_bytes = static_cast<size_t>(tt) * NRT * WT * pitch;
                const size_t partial_bytes = static_cast<size_t>(nw) * 8 * 1024;        // the split-K partial sums of one timestep
                if (wk_log2 > 0 && tiles_bytes < partial_bytes) tiles_bytes = partial_bytes;
                const size_t bytes = tiles_bytes + stage_bytes;
                if (bytes > lds_cap) continue;
                if (sc * groups * NRT * (WT / 2) > max_items) continue;
                const bool full_width = tw == g0.Wo;
                int run = 0;
                for (int cand : {8, 4}) {
                    if (cand > vec || run != 0) continue;
                    if (full_width ? ((th * g0.Wo) % cand == 0) : (tw % cand == 0 && g0.Wo % cand == 0)) run = cand;
                }
                // `all_full`: every tile is whole and made of whole runs (runs never straddle two images of a tile).
                const bool all_full = g0.Ho % th == 0 && g0.Wo % tw == 0 && run != 0 && (th * tw) % run == 0 && g0.N % ti == 0;
                const double work = static_cast<double>(img_groups) * tiles_x * tiles_y * oc_tiles;
                const double lane_eff = static_cast<double>(g0.N) * g0.Ho * g0.Wo / (static_cast<double>(img_groups) * tiles_x * tiles_y * PT);
                const double waves = work < cus ? 1.0 : static_cast<double>(static_cast<long long>((work + cus - 1) / cus));
                const double fill = work / (waves * cus);
                const double halo = static_cast<double>(NR) * WT / (static_cast<double>(th) * tw);   // per image
                double score = lane_eff * oc_eff * fill / (1.0 + 0.1 * (halo - 1.0)) / (1.0 + 0.05 * (oc_tiles - 1));
                score /= 1.0 + 0.08 * ((1 << wk_log2) - 1);
                if (run == 0) score *= 0.4;        // element-wise 2-byte stores are very slow
                else if (!all_full) score *= 0.8;  // the masked variant
                else if (run == 4) score *= 0.95;
                if (score > best) {
                    best = score;
                    best_plan = MmPlan{th, tw, tiles_x, tiles_y, NR, WT, wm_log2, wn_log2, wk_log2, oc_tiles, run, all_full ? 1 : 0,
                                       static_cast<int>(tiles_bytes), sc, pitch, bytes, nw, score, ti};
                }
              }
            }
        }
    }
    return best > 0.0;
}

bool plan_mm(const ConvGeom& g, int tt, int load_mode, int vec, int nw, MmPlan& out) {
    using Key = std::tuple<int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int>;
    static std::mutex mu;
    static std::map<Key, std::pair<bool, MmPlan>> plans;
    const Key key(g.N, g.H, g.W, g.KH, g.KW, g.sh, g.sw, g.ph, g.pw, g.pitch, g.Cout, g.npairs, g.nchunks, tt, load_mode, vec, nw);
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = plans.find(key);
        if (it != plans.end()) {
            out = it->second.second;
            return it->second.first;
        }
    }
    MmPlan p = {};
    const bool ok = plan_mm_uncached(g, tt, load_mode, vec, nw, p);
    std::lock_guard<std::mutex> lock(mu);
    plans[key] = std::make_pair(ok, p);
    out = p;
    return ok;
}

bool plan(const ConvGeom& g, int t_in, int tt, int load_mode, bool want_vec8, Plan& out) {
    using Key = std::tuple<int, int, int, int, int, int, int, int, int, int, int, int, int, int, int>;
    static std::mutex mu;
    static std::map<Key, std::pair<bool, Plan>> plans;
    const Key key(g.N, g.H, g.W, g.KH, g.KW, g.sh, g.sw, g.ph, g.pw, g.pitch, g.Cout, t_in, tt, load_mode,
                  want_vec8 ? 1 : 0);
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = plans.find(key);
        if (it != plans.end()) {
            out = it->second.second;
            return it->second.first;
        }
    }
    Plan p = {};
    const bool ok = plan_uncached(g, t_in, tt, load_mode, want_vec8, p);
    std::lock_guard<std::mutex> lock(mu);
    plans[key] = std::make_pair(ok, p);
    out = p;
    return ok;
}

}  // namespace
}  // namespace snnf

namespace snnf {
char* conv_plan_buffer() {
    static thread_local char buffer[256] = {0};
    return buffer;
}
}  // namespace snnf

extern "C" const char* snnf_conv_last_plan(void) { return snnf::conv_plan_buffer(); }

namespace snnf {
namespace {
// Shared body of snnf_conv_lif and snnf_conv_bias. `analog_out`: no neuron - the convolution output (+ bias, + residual)
// is written in the activation dtype where the spikes would go, and no membrane is read or written.
int conv_lif_impl(const void* const* xs, const void* const* residuals, int T, int N, int Cin, int H, int W,
                  int x_dtype, const void* packed_weight, int Cout, int KH, int KW, int stride_h, int stride_w,
                  int pad_h, int pad_w, const void* v_init, int v_dtype, void* spikes,
                  int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset, float tau,
                  void* stream, bool analog_out, bool x_rowbits = false, bool out_rowbits = false) {
    if (xs == nullptr || packed_weight == nullptr || spikes == nullptr || (v_out == nullptr && !(out_rowbits && T <= SNNF_MAX_T_PER_LAUNCH)))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_lif: xs, packed_weight, spikes and v_out must be non-null");
    if (T < 1 || N < 1 || Cin < 1 || H < 1 || W < 1 || Cout < 1 || KH < 1 || KW < 1 || stride_h < 1 || stride_w < 1 ||
        pad_h < 0 || pad_w < 0)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_lif: bad extent (T=%d N=%d Cin=%d H=%d W=%d Cout=%d K=%dx%d s=%dx%d p=%dx%d)",
                    T, N, Cin, H, W, Cout, KH, KW, stride_h, stride_w, pad_h, pad_w);
    if (!valid_dtype(x_dtype) || !valid_dtype(v_dtype)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_lif: unknown dtype code");
    if (v_dtype != SNNF_F32 && v_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: unsupported_dtype: membrane dtype must be fp32 or the activation dtype");
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: unsupported_tau: tau must be nonzero");
    if (H + 2 * pad_h < KH || W + 2 * pad_w < KW)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: unsupported_kernel: kernel larger than padded input");
    if (2 * pad_h > KH || 2 * pad_w > KW)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: unsupported_padding: padding %dx%d too large for kernel %dx%d", pad_h, pad_w, KH, KW);
    if (!aligned_to(packed_weight, 16)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_lif: packed_weight must be 16-byte aligned");
    for (int t = 0; t < T; ++t) {
        if (xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_lif: xs[%d] is null", t);
        if (residuals != nullptr && residuals[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_lif: residuals[%d] is null", t);
    }
    const int Ho_real = (H + 2 * pad_h - KH) / stride_h + 1;
    const int Wo_real = (W + 2 * pad_w - KW) / stride_w + 1;
    if (static_cast<int64_t>(N) * Cin * H * W >= (1LL << 30) || static_cast<int64_t>(N) * Cout * Ho_real * Wo_real >= (1LL << 31))
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: unsupported_shape: more than 2^30 input elements per timestep");

    ConvGeom g = {};
    g.N = N; g.Cin = Cin; g.Cout = Cout; g.KH = KH; g.KW = KW;
    g.sh = stride_h; g.sw = stride_w; g.ph = pad_h; g.pw = pad_w;
    const bool pointwise = KH == 1 && KW == 1 && stride_h == 1 && stride_w == 1 && pad_h == 0 && pad_w == 0;
    if (pointwise) {
        // A pointwise convolution has no spatial structure: treat each image as one row of H * W pixels.
        g.H = 1; g.W = H * W;
    } else {
        g.H = H; g.W = W;
    }
    g.Ho = (g.H + 2 * pad_h - KH) / stride_h + 1;
    g.Wo = (g.W + 2 * pad_w - KW) / stride_w + 1;
    const PackGeom pg = make_pack_geom(Cout, Cin, KH, KW, x_dtype == SNNF_F32);
    g.CK = pg.CK; g.nchunks = pg.nchunks; g.npairs = pg.npairs; g.nchunks_r = pg.nchunks_r;
    g.groups_log2 = 0;
    while ((8 << g.groups_log2) < pg.CK) ++g.groups_log2;
    g.pitch = pg.CK * 2 + 16;
    g.spike_step_stride = spike_step_stride;
    g.v_is_f32 = v_dtype == SNNF_F32 ? 1 : 0;
    g.analog_out = analog_out ? 1 : 0;
    const int xsize = dtype_size(x_dtype);
    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    hipStream_t hs = as_stream(stream);

    constexpr int kMaxTT = 4;
    bool all_shared = T > 1;
    bool pair_aligned = xsize == 2 && (g.W % 2 == 0);
    // 8 consecutive output pixels start 16-byte aligned whenever their first pixel offset is a multiple of 8.
    bool vec_ok = ((static_cast<int64_t>(g.Ho) * g.Wo) % 8 == 0) && (spike_step_stride % 8 == 0) && aligned_to(spikes, 16) &&
                  aligned_to(v_out, 16) && (v_init == nullptr || aligned_to(v_init, 16));
    // The same for runs of 4 pixels (8-byte spike accesses, 16-byte membrane accesses).
    bool vec4_ok = ((static_cast<int64_t>(g.Ho) * g.Wo) % 4 == 0) && (spike_step_stride % 4 == 0) && aligned_to(spikes, 8) &&
                   aligned_to(v_out, 16) && (v_init == nullptr || aligned_to(v_init, 16)) && xsize == 2;
    for (int t = 0; t < T; ++t) {
        all_shared = all_shared && xs[t] == xs[0];
        pair_aligned = pair_aligned && aligned_to(xs[t], 4);
        if (residuals != nullptr) vec_ok = vec_ok && aligned_to(residuals[t], 16);
        if (residuals != nullptr) vec4_ok = vec4_ok && aligned_to(residuals[t], 8);
    }
    const int load_mode = xsize == 4 ? LOAD_2XF32 : (pair_aligned ? LOAD_PAIR32 : LOAD_2X16);
    // The matrix kernel also pairs the pixels of planes of odd width (2 columns or more): 4-byte loads at 2-byte alignment.
    const int mm_load_mode = (xsize == 2 && g.W % 2 == 1 && g.W >= 3) ? LOAD_PAIR32 : load_mode;

    // Kernel choice. Layers whose arithmetic intensity is far below the matrix-core / HBM ridge (about 300 flop/byte)
    // run the time-outer kernel (small footprint, two workgroups per CU, membrane resident for any T); the others
    // accumulate up to 4 timesteps side by side so that each weight fragment load feeds 4x the matrix work.
    const double flops = 2.0 * (all_shared ? 1 : T) * N * static_cast<double>(Ho_real) * Wo_real * Cout * Cin * KH * KW;
    const double bytes = static_cast<double>(xsize) * ((all_shared ? 1 : T) * static_cast<double>(N) * Cin * H * W +
                                                       static_cast<double>(T) * N * Cout * Ho_real * Wo_real) +
                         4.0 * N * Cout * Ho_real * Wo_real;
    // Dense layers whose input channels fill whole groups of 8 (or fit a single group) go to the 8-wave matrix kernel
    // whatever their intensity (its per-tile cost is the lower one); pointwise layers stay with the pointwise kernel unless
    // they are compute bound (deep 512 -> 512 layers: an image is then one row of H * W pixels to the matrix kernel).
    // Measured on 1x1 layers of more than one channel chunk (T = 4, us on the pointwise / the matrix kernel): 256 -> 256 at 28^2
    // x 32 images (128 MB) 79 / 55, 256 -> 512 at 28^2 x 16 (103 MB) 78 / 51, 192 -> 64 at 28^2 x 32 (58 MB) 57 / 32, 384 -> 96 at
    // 14^2 x 32 (26 MB) 42 / 36, 1024 -> 64 at 8^2 x 8 56 / 54, but 256 -> 128 at 56^2 x 32 (360 MB) 90 / 139: the pointwise
    // kernel keeps the layers that are mostly memory traffic.
    // Row-packed spikes in (`x_rowbits`): xs[t] are [N][Cin][H * W / 8] bytes; only the pointwise kernel's fast variant reads them.
    if (x_rowbits) {
        const bool fast_neuron = lif.charge_mode == CHARGE_SCALE && !lif.soft_reset;
        if (!pointwise || residuals != nullptr || xsize != 2 || v_dtype != SNNF_F32 || !fast_neuron || Cin % 8 != 0 || Cout % 32 != 0 ||
            g.Wo % 64 != 0 || !vec_ok || static_cast<int64_t>(Cout) * g.Wo >= (1LL << 30))
            return fail(SNNF_ERR_UNSUPPORTED, "snnf_pwconv_lif_rowbits: unsupported_shape: needs a 1x1 stride-1 layer without residual, 16-bit "
                        "operands, an fp32 membrane, the common neuron (tau a power of two above 1, hard reset), Cin %% 8 == 0, Cout %% 32 == 0, "
                        "H * W %% 64 == 0 and 16-byte aligned outputs");
        all_shared = false;
    } else if (out_rowbits) {
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_pwconv_lif_rowbits: row-packed output needs row-packed input");
    }
    g.bits_out = out_rowbits ? 1 : 0;
    const bool pointwise_to_matrix = !x_rowbits && pointwise && (flops / bytes >= 200.0 || (Cin > 128 && bytes < 200.0e6));
    // A neuron-free pointwise layer (snnf_conv_bias) has no other kernel to go to: the pointwise kernel always runs a neuron.
    const bool matrix_candidate = (!pointwise || pointwise_to_matrix || (analog_out && !x_rowbits)) && (Cin % 8 == 0 || Cin < 8);
    int window = 0;
    Plan pl = {};
    bool planned = false;
    bool pw_kernel = false;
    bool mm_kernel = false;
    MmPlan mp = {};
    if (matrix_candidate) {
        // 8-wave matrix kernel: the largest window of 4, 2 or 1 timesteps whose halo tiles fit LDS.
        // One analog frame for all T: a single stage of input (TT = 1), up to 16 LIF steps per launch.
        int w2 = 1;
        while (!all_shared && w2 < T && w2 < kMaxTT) w2 *= 2;
        const bool fast_layer = Cout % 64 == 0 && v_dtype == SNNF_F32 && lif.charge_mode == CHARGE_SCALE && !lif.soft_reset;
        const int vec = vec_ok ? 8 : (vec4_ok ? 4 : 0);
        for (; w2 >= 1 && !mm_kernel; w2 >>= 1) {
            MmPlan p8 = {}, p4 = {};
            const bool ok8 = plan_mm(g, w2, mm_load_mode, vec, 8, p8);
            // One shared frame: a single short matrix stage, then T steps of epilogue per tile. Two 4-wave workgroups per
            // CU (fast variant only) overlap one's epilogue with the other's loads and matrix work; measured 15 % faster on
            // a 7x7/2 stem, slower on every layer with a deep matrix loop.
            const bool ok4 = all_shared && fast_layer && plan_mm(g, w2, mm_load_mode, vec, 4, p4) && p4.all_full && p4.run >= 4;
            if (!ok8 && !ok4) continue;
            mp = ok4 ? p4 : p8;
            // The masked variant with 4 timesteps of accumulators spills registers (and every reload then waits behind
            // the activation prefetch): it runs windows of 2.
            const bool fast_plan = fast_layer && mp.all_full && mp.run >= 4;
            if (w2 == 4 && !fast_plan) continue;
            mm_kernel = planned = true;
            window = w2;
        }
        if (mm_kernel && all_shared) window = T < SNNF_MAX_T_PER_LAUNCH ? T : SNNF_MAX_T_PER_LAUNCH;
        if (mm_kernel) {
            pl.TH = mp.TH; pl.TW = mp.TW; pl.tiles_x = mp.tiles_x; pl.tiles_y = mp.tiles_y; pl.NR = mp.NR; pl.WT = mp.WT;
            pl.wm_log2 = mp.wm_log2; pl.wn_log2 = mp.wn_log2; pl.oc_tiles = mp.oc_tiles; pl.lds_bytes = mp.lds_bytes;
        }
    }
    if (analog_out && !mm_kernel)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_bias: unsupported_shape: only layers the 8-wave matrix kernel takes "
                    "(Cin %% 8 == 0 or Cin < 8, tiles that fit LDS)");
    // Everything else: the time-outer kernels for a shared frame or a low intensity, the 4-wave T-in-M kernel otherwise.
    bool time_outer = !mm_kernel && (all_shared || x_rowbits || flops / bytes < 200.0);
    // Pointwise kernel: where the weight fragments live (registers only in the fast variant) and the LDS that takes.
    auto pw_config = [&](bool allow_regs, ConvGeom& gg) -> size_t {
        const size_t xb = static_cast<size_t>(64) * gg.pitch;
        const size_t wbytes = static_cast<size_t>(4) * gg.nchunks * gg.npairs * kFragBytes;
        size_t bytes = xb + kPwStageBytes;
        gg.x_bufs = 1;
        gg.w_lds = 0;   // streamed from L2
        if (allow_regs && gg.nchunks == 1 && gg.npairs == 8) {
            gg.w_lds = 2;   // a wave's 8 fragments in registers
        } else if ((bytes + wbytes) * 2 <= kMaxLds) {
            gg.w_lds = 1;   // the workgroup's fragments in LDS, two workgroups per CU
            bytes += wbytes;
        }
        if ((bytes + xb) * 2 <= kMaxLds) {
            gg.x_bufs = 2;
            bytes += xb;
        }
        return bytes;
    };
    if (time_outer && pointwise && Cin % 8 == 0 && static_cast<int64_t>(Cout) * g.Wo < (1LL << 30)) {
        // Pointwise kernel: flat tiles of 64 pixels x 128 output channels, no planning needed.
        pw_kernel = planned = true;
        window = T < SNNF_MAX_T_PER_LAUNCH ? T : SNNF_MAX_T_PER_LAUNCH;
        pl.TH = 1; pl.TW = 64; pl.tiles_x = (g.Wo + 63) / 64; pl.tiles_y = N; pl.NR = 1; pl.WT = 64;
        pl.wm_log2 = 0; pl.wn_log2 = 2; pl.oc_tiles = (Cout + 127) / 128;
        pl.lds_bytes = 0;
    } else if (time_outer) {
        planned = plan(g, 1, 0, load_mode, vec_ok, pl);
        window = T < SNNF_MAX_T_PER_LAUNCH ? T : SNNF_MAX_T_PER_LAUNCH;
        if (!planned) time_outer = false;
    }
    if (!time_outer && !mm_kernel) {
        // Timesteps per launch: as many (<= 4) as fit LDS side by side; a shared analog frame needs one tile for any window.
        window = T < kMaxTT ? T : kMaxTT;
        int w2 = 1;
        while (w2 < window) w2 *= 2;
        window = w2;
        while (true) {
            planned = plan(g, all_shared ? 1 : window, window, load_mode, vec_ok, pl);
            if (planned || window == 1) break;
            window >>= 1;
        }
    }
    if (!planned)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: unsupported_shape: no activation tile fits LDS (W=%d, kernel %dx%d, stride %dx%d)",
                    W, KH, KW, stride_h, stride_w);
    g.TH = pl.TH; g.TW = pl.TW; g.tiles_x = pl.tiles_x; g.tiles_y = pl.tiles_y; g.NR = pl.NR; g.WT = pl.WT;
    g.wm_log2 = pl.wm_log2; g.wn_log2 = pl.wn_log2; g.oc_tiles = pl.oc_tiles;
    g.vec8 = vec_ok ? 1 : 0;
    g.d_TW = make_fast_div(g.TW); g.d_Ho = make_fast_div(g.Ho); g.d_H = make_fast_div(g.H);
    g.d_WTP = make_fast_div(g.WT / 2); g.d_stage_rows = make_fast_div(g.NR * (g.WT / 2));
    g.d_tiles_x = make_fast_div(g.tiles_x); g.d_oc_tiles = make_fast_div(g.oc_tiles);
    {   // Matrix kernel: which operand an XCD's L2 should keep (see the kernel's tile walk).
        const int64_t weight_bytes = static_cast<int64_t>(Cout) * Cin * KH * KW * 2;
        const int64_t act_bytes = static_cast<int64_t>(all_shared ? 1 : window) * N * Cin * H * W * dtype_size(x_dtype);
        if (mm_kernel && g.oc_tiles % 8 == 0 && weight_bytes > act_bytes) {
            g.oc_major = 1;
            g.d_oc_tiles = make_fast_div(g.oc_tiles / 8);
        }
    }
    g.tiles_img = g.tiles_x * g.tiles_y; g.d_tiles_img = make_fast_div(g.tiles_img); g.d_KW = make_fast_div(g.KW);
    g.run8 = mm_kernel ? mp.run : 0;
    g.wk_log2 = mm_kernel ? mp.wk_log2 : 0;
    g.mm_stage_off = mm_kernel ? mp.stage_off : 0;
    g.stage_chunks = mm_kernel ? mp.stage_chunks : 1;
    if (mm_kernel) g.pitch = mp.pitch;
    g.d_npairs = make_fast_div(g.npairs);
    g.TI = mm_kernel ? mp.TI : 1;
    g.img_groups = (g.N + g.TI - 1) / g.TI;
    g.d_NR = make_fast_div(g.NR);
    g.d_tile_px = make_fast_div(g.TH * g.TW);
    if (mm_kernel) g.d_stage_rows = make_fast_div(g.TI * g.NR * (g.WT / 2));

    size_t lds_bytes = pl.lds_bytes;
    if (time_outer && !pw_kernel) {
        // Keep the workgroup's weight fragments in LDS when two workgroups per CU still fit: the matrix loop then needs
        // no global loads at all.
        const size_t wbytes = (static_cast<size_t>(1) << g.wn_log2) * 1 * g.nchunks * g.npairs * kFragBytes;
        if ((lds_bytes + wbytes) * 2 <= kMaxLds) {
            g.w_lds = 1;
            lds_bytes += wbytes;
        }
    }
    const int cu_per_xcd = (compute_units() + 7) / 8;
    auto grid_for = [&](const ConvGeom& gg, int per_cu) {
        const int px_tiles = mm_kernel ? gg.img_groups * gg.tiles_img : gg.tiles_x * gg.tiles_y;
        const int work_per_xcd = gg.oc_major ? px_tiles * (gg.oc_tiles / 8) : ((px_tiles + 7) / 8) * gg.oc_tiles;
        int slots = cu_per_xcd * per_cu;
        if (slots > work_per_xcd) slots = work_per_xcd;
        return slots * 8;
    };
    const int per_cu = mm_kernel ? 8 / mp.nw : (time_outer ? 2 : ((pl.lds_bytes * 2 <= kMaxLds && window < 4) ? 2 : 1));

    // Pointwise layers: the fast variant takes the tiles that lie inside their image when the layer qualifies (common
    // neuron, aligned outputs, fp32 membrane, whole channel fragments); the general variant takes the ragged last tile of
    // each image, or everything.
    struct Part { ConvGeom g; size_t lds; int tt; };
    Part parts[2];
    int nparts = 0;
    if (pw_kernel) {
        const int P = g.Wo;
        const bool fast_ok = lif.charge_mode == CHARGE_SCALE && !lif.soft_reset && vec_ok && Cout % 32 == 0 && v_dtype == SNNF_F32;
        const int full_tiles = fast_ok ? P / 64 : 0;
        if (full_tiles > 0) {
            Part& f = parts[nparts++];
            f.g = g; f.tt = -2;
            f.g.tiles_x = full_tiles; f.g.px_base = 0;
            // Outputs that the caches cannot hold anyway are streamed past L2, which then keeps the activation tiles for
            // their second pass (the other output-channel tile). Smaller outputs stay cached for the layer that reads them.
            const int64_t out_bytes = out_rowbits ? static_cast<int64_t>(N) * Cout * P * (v_out != nullptr ? 4 : 0)
                                                  : static_cast<int64_t>(N) * Cout * P * (static_cast<int64_t>(window) * dtype_size(x_dtype) + 4);
            f.g.stream_out = out_bytes >= kStreamOutBytes ? 1 : 0;
            f.g.d_tiles_x = make_fast_div(full_tiles);
            f.lds = pw_config(true, f.g);
        }
        if (full_tiles * 64 < P) {
            Part& r = parts[nparts++];
            r.g = g; r.tt = -1;
            r.g.tiles_x = (P - full_tiles * 64 + 63) / 64; r.g.px_base = full_tiles * 64;
            r.g.d_tiles_x = make_fast_div(r.g.tiles_x);
            r.lds = pw_config(false, r.g);
        }
    } else if (mm_kernel) {
        const bool fast_ok = mp.all_full && mp.run >= 4 && Cout % 64 == 0 && v_dtype == SNNF_F32 &&
                             lif.charge_mode == CHARGE_SCALE && !lif.soft_reset;   // = fast_plan above
        parts[0].g = g; parts[0].lds = lds_bytes; parts[0].tt = (mp.nw == 4 ? 30 : (fast_ok ? 20 : 10)) + (all_shared ? 1 : window);
        nparts = 1;
    } else {
        parts[0].g = g; parts[0].lds = lds_bytes; parts[0].tt = time_outer ? 0 : window;
        nparts = 1;
    }

    snprintf(snnf::conv_plan_buffer(), 256,
             "kernel=%s variant=%d window=%d launches=%d tile=%dx%dx%d halo=%dx%d waves=%dx%dx%d oc_tiles=%d px_tiles=%d "
             "stage_chunks=%d run=%d lds=%zu grid=%d",
             pw_kernel ? "pointwise" : (mm_kernel ? "matrix" : (time_outer ? "time_outer" : "t_in_m")), parts[0].tt, window,
             nparts * ((T + window - 1) / window), g.TI, g.TH, g.TW, g.NR, g.WT, 1 << g.wm_log2, 1 << g.wn_log2, 1 << g.wk_log2,
             g.oc_tiles, mm_kernel ? g.img_groups * g.tiles_img : g.tiles_x * g.tiles_y, g.stage_chunks, g.run8, parts[0].lds,
             grid_for(parts[0].g, per_cu));
    for (int t0 = 0; t0 < T; t0 += window) {
        const int tw = (T - t0) < window ? (T - t0) : window;
        ConvLaunch L = {};
        for (int t = 0; t < window; ++t) {
            L.xs.p[t] = xs[t0 + (t < tw ? t : 0)];  // padded steps repeat step 0 and are never stored
            if (residuals != nullptr) L.residuals.p[t] = residuals[t0 + (t < tw ? t : 0)];
        }
        L.has_residual = residuals != nullptr ? 1 : 0;
      for (int part = 0; part < nparts; ++part) {
        L.g = parts[part].g;
        L.g.T = tw;
        L.g.shared_x = (all_shared && (window > 1 || time_outer)) ? 1 : 0;
        L.wpacked = static_cast<const uint16_t*>(packed_weight);
        L.bias = reinterpret_cast<const float*>(L.wpacked + packed_weight_elems(pg));
        L.v_init = t0 == 0 ? v_init : v_out;
        L.spikes = static_cast<char*>(spikes) + static_cast<int64_t>(t0) * spike_step_stride * (out_rowbits ? 1 : xsize);
        L.v_out = v_out;
        L.lif = lif;
        L.grid = grid_for(L.g, per_cu);
        L.lds_bytes = parts[part].lds;
        L.stream = hs;
        int rc;
        const int tt = parts[part].tt;
        const int lm = x_rowbits ? static_cast<int>(LOAD_ROWBITS) : (mm_kernel ? mm_load_mode : load_mode);
        if (x_dtype == SNNF_F32) rc = launch_conv_f32(L, tt, lm);
        else if (x_dtype == SNNF_BF16) rc = launch_conv_bf16(L, tt, lm);
        else rc = launch_conv_f16(L, tt, lm);
        if (rc != SNNF_OK) return rc;
      }
    }
    return SNNF_OK;
}
}  // namespace
}  // namespace snnf

extern "C" int snnf_conv_lif(const void* const* xs, const void* const* residuals, int T, int N, int Cin, int H, int W,
                             int x_dtype, const void* packed_weight, int Cout, int KH, int KW, int stride_h, int stride_w,
                             int pad_h, int pad_w, const void* v_init, int v_dtype, void* spikes,
                             int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset, float tau,
                             void* stream) {
    return snnf::conv_lif_impl(xs, residuals, T, N, Cin, H, W, x_dtype, packed_weight, Cout, KH, KW, stride_h, stride_w, pad_h,
                               pad_w, v_init, v_dtype, spikes, spike_step_stride, v_out, v_threshold, v_reset, tau, stream, false);
}

extern "C" int snnf_pwconv_lif_rowbits(const void* const* xs_bits, int T, int N, int Cin, int H, int W, int x_dtype,
                                       const void* packed_weight, int Cout, const void* v_init, void* spikes, int spikes_packed,
                                       int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset, float tau,
                                       void* stream) {
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return snnf::fail(SNNF_ERR_UNSUPPORTED, "snnf_pwconv_lif_rowbits: unsupported_dtype: the matrix operands are bf16 or fp16");
    return snnf::conv_lif_impl(xs_bits, nullptr, T, N, Cin, H, W, x_dtype, packed_weight, Cout, 1, 1, 1, 1, 0, 0, v_init, SNNF_F32, spikes,
                               spike_step_stride, v_out, v_threshold, v_reset, tau, stream, false, true, spikes_packed != 0);
}

extern "C" int snnf_conv_bias(const void* const* xs, const void* const* residuals, int T, int N, int Cin, int H, int W,
                              int x_dtype, const void* packed_weight, int Cout, int KH, int KW, int stride_h, int stride_w,
                              int pad_h, int pad_w, void* out, int64_t out_step_stride, void* stream) {
    // The neuron parameters only steer the variant selection (the common neuron qualifies for the fast variant).
    return snnf::conv_lif_impl(xs, residuals, T, N, Cin, H, W, x_dtype, packed_weight, Cout, KH, KW, stride_h, stride_w, pad_h,
                               pad_w, nullptr, SNNF_F32, out, out_step_stride, out, 1.0f, 0.0f, 2.0f, stream, true);
}
