// Dense convolution + bias (+ residual) + LIF over up to 4 timesteps side by side, for layers bound by the matrix
// cores (3x3 and larger kernels with tens to hundreds of channels).
//
// Same implicit GEMM as snnf_conv_kernel.h (M = output channels, N = pixels, K = taps x channels, packed weights), built
// around what limits such a kernel on this machine:
//   * 8 waves per workgroup, one workgroup per CU: two waves per SIMD, so that one wave's operand reads, LIF epilogue and
//     stores overlap the other's matrix instructions. A wave owns 64 channels x 32 pixels x TT timesteps (8 accumulator
//     tiles, 128 registers): a weight fragment feeds TT matrix instructions, an activation fragment two.
//   * A tile is TH x TW output pixels of ONE image, so a lane's pixel, its LDS address and its output offset are kernel
//     constants; a tile contributes uniform bases only. The halo tile in LDS holds explicit zeros for padding, so the
//     matrix loop has no bounds logic: per pair of k-slots the (tap, channel group) offsets are walked on the scalar unit.
//   * Staging loads are unconditional (out-of-image items read a valid address and are zeroed on their way into LDS)
//     and issued from a single place one stage ahead; the LIF epilogue runs on a wave-private LDS stage, 16 channel rows
//     x 32 pixels at a time, so that a lane owns 8 consecutive pixels: 16-byte spike stores, membrane in registers
//     across the TT steps.
//   * SK: layers with few pixels and many channels (deep stages) do not fill the machine with 64 x 32 wave tiles, so
//     WK waves share an output tile, each taking every WK-th pair of k-slots, and add their sums through LDS.
// FAST: every tile is full, runs of 8 pixels are contiguous and 16-byte aligned, Cout % 64 == 0, fp32 membrane, the
// common neuron (power-of-two tau, hard reset); the general variant masks pixels and rows and takes any neuron. Requires whole
// channel groups (Cin % 8 == 0) or Cin < 8. With TT == 1 the single stage may be one analog frame shared by all g.T
// timesteps: it is convolved once.
#pragma once

#include "snnf_conv_pw_kernel.h"

namespace snnf {

constexpr int kMmStagePitch = 40;                          // floats per channel row of a wave's stage (32 pixels + padding)
constexpr int kMmStageFloats = 16 * kMmStagePitch;         // 16 channel rows
static_assert(kMmStageFloats * sizeof(float) == kMmStageBytesPerWave, "host and kernel disagree on the stage size");
// Spatial staging items per thread and stage: 64 prefetch registers whatever the load mode and the timesteps per stage.
// The split-K variants stage deep layers with small tiles and are short of registers (with the full 64 prefetch registers
// they spilled 30-140): with paired loads and 2 or 4 timesteps per stage they take half the slots, i.e. smaller LDS
// stages (the unpaired load mode has half the slots to begin with and is better off with the larger stages).
__host__ __device__ constexpr int mm_staging_slots(int load_mode, int tt, bool split_k = false) {
    const int slots = (load_mode == LOAD_PAIR32 ? 8 : 4) / tt;
    return (split_k && load_mode == LOAD_PAIR32 && tt >= 2) ? slots / 2 : slots;
}
typedef float cv_f32x4 __attribute__((ext_vector_type(4)));

// NW waves per workgroup: 8 (one workgroup per CU) or 4 (two independent workgroups per CU, whose load, matrix and
// epilogue phases overlap each other instead of running in lockstep across the whole CU).
template <typename XT, int TT, int LM, bool FAST, bool SK, int NW>
__global__ __launch_bounds__(NW * 64, 8 / NW) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_mm_lif_kernel(
    const StepPtrs xs, const StepPtrs residuals, const int has_residual, const ConvGeom g,
    const uint16_t* __restrict__ wpacked, const float* __restrict__ bias, const void* __restrict__ v_init,
    XT* __restrict__ spikes, void* __restrict__ v_out, const LifParams lif) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    constexpr int RPE = LM == LOAD_PAIR32 ? 1 : 2;
    constexpr int SS = mm_staging_slots(LM, TT, SK);
    constexpr uint32_t ES = static_cast<uint32_t>(sizeof(XT));
    constexpr int NT = NW * 64;                               // threads per workgroup
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int l32 = lane & 31;
    const int wm = wave & ((1 << g.wm_log2) - 1);
    const int wn = (wave >> g.wm_log2) & ((1 << g.wn_log2) - 1);
    const int wk = SK ? (wave >> (g.wm_log2 + g.wn_log2)) : 0;     // K slice of this wave (split-K variant)
    const int WK = SK ? (1 << g.wk_log2) : 1;

    const int groups = 1 << g.groups_log2;                   // channel groups of 8 per packed chunk
    const int stage_groups = groups * g.stage_chunks;        // ... per LDS stage (a stage holds stage_chunks chunks)
    // fp32 tensors (see kSplitParts): a stage holds stage_chunks REAL channel chunks, fetched once and written to LDS as their
    // high and their low bf16 terms side by side ([hi: stage channels][lo: stage channels] per pixel); the matrix steps of a
    // stage then run the three parts of the packed weight against them (w_hi on hi, w_lo on hi, w_hi on lo).
    constexpr int PARTS = LM == LOAD_2XF32 ? kSplitParts : 1;
    const int nstages = (g.nchunks_r + g.stage_chunks - 1) / g.stage_chunks;
    const int lo_off = g.stage_chunks * g.CK * 2;            // bytes from a pixel's high terms to its low terms
    const int WTP = g.WT >> 1;
    const int rows_all = g.TI * g.NR;                        // halo rows of the TI images of a tile, stacked
    const int tile_px = g.TH * g.TW;                         // output pixels per image and tile
    const int tile_bytes = rows_all * g.WT * g.pitch;        // one timestep's halo tile(s)
    float* __restrict__ stage = reinterpret_cast<float*>(lds + g.mm_stage_off) + wave * kMmStageFloats;
    // The workgroup's bias values (its 64 x WN output channels) are fetched with the first loads of a tile and parked in LDS
    // until the epilogue, which would otherwise wait for them from memory group by group.
    float* __restrict__ bias_lds = reinterpret_cast<float*>(lds + g.mm_stage_off) + NW * kMmStageFloats;
    // fp32 tensors: set by any thread that stages a non-zero low term (activations that are exact in bf16, spikes above all,
    // have none: the third part of the matrix steps is then skipped for the stage). One word behind the bias values.
    volatile int& stage_has_low_terms = *reinterpret_cast<volatile int*>(bias_lds + 512);
    float bias_pre = 0.0f;
    auto fetch_bias = [&](int oc_t) __attribute__((always_inline)) {
        const int oc = (oc_t << g.wn_log2) * 64 + tid;
        bias_pre = (tid < (64 << g.wn_log2) && oc < g.Cout) ? bias[oc] : 0.0f;
    };
    const int nocf = (g.Cout + 31) >> 5;
    const int total_pairs = g.nchunks * g.npairs;
    const int64_t frag_stride_ocf = static_cast<int64_t>(total_pairs) * (kFragBytes / 2);
    const int64_t plane = static_cast<int64_t>(g.H) * g.W;
    const int po = g.Ho * g.Wo;
    const bool pair_shift = LM == LOAD_PAIR32;               // tile columns start at an even input column

    // ---- kernel constants of the staging: item e = (channel group, tile row, column pair).
    int item_cg[SS], item_r[SS], item_c[SS], item_i[SS];     // item_cg < 0: idle slot; item_i: image of the tile
    uint32_t item_dst[SS];
    int item_src[SS];                                        // element offset of (image i, channel cg * 8, row r, column 2 cp) from the tile origin
    const int image_elems = g.Cin * g.H * g.W;
#pragma unroll
    for (int s = 0; s < SS; ++s) {
        const int e = s * NT + tid;
        const int cg = fast_div(e, g.d_stage_rows);
        const int rem = e - cg * (rows_all * WTP);
        const int rr = fast_div(rem, g.d_WTP);               // stacked row
        const int cp = rem - rr * WTP;
        const int ii = fast_div(rr, g.d_NR);
        const int r = rr - ii * g.NR;
        item_cg[s] = cg < stage_groups ? cg : -1;
        item_r[s] = r;
        item_i[s] = ii;
        item_c[s] = 2 * cp;
        item_dst[s] = static_cast<uint32_t>((rr * g.WT + 2 * cp) * g.pitch + cg * 16);
        item_src[s] = ii * image_elems + (cg * 8 * g.H + r) * g.W + 2 * cp;
    }

    const int last_channel = g.Cin < 8 ? g.Cin - 1 : 7;
    const int taps = g.KH * g.KW;
    // ---- the stage in flight.
    uint32_t pre[SS][TT][8][RPE];
    uint32_t pre_zero0 = 0, pre_zero1 = 0;                   // bit s: first / second column of item s is padding or beyond Cin

    // Loads of stage `stg` (stage_chunks channel chunks) of the tile whose halo starts at input (row ih_lo, column iw_lo)
    // of image n.
    auto issue_loads = [&](int stg, int n, int ih_lo, int iw_lo) __attribute__((always_inline)) {
        const int chunk = stg * g.stage_chunks;                                                  // first (real) chunk of the stage
        const int64_t origin = (static_cast<int64_t>(n) * g.Cin + chunk * g.CK) * plane;     // elements, always inside the tensor
        const int tile_rel = ih_lo * g.W + iw_lo;                                               // may be negative
        uint32_t off0[SS], off1[SS];
        uint32_t z0 = 0, z1 = 0;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            const int ih = ih_lo + item_r[s];
            const int iw = iw_lo + item_c[s];
            const bool cok = item_cg[s] >= 0 && chunk * g.CK + item_cg[s] * 8 < g.Cin && ih >= 0 && ih < g.H && n + item_i[s] < g.N;
            const bool ok0 = cok && iw >= 0 && iw < g.W;
            const bool ok1 = cok && iw + 1 >= 0 && iw + 1 < g.W;
            const uint32_t src = static_cast<uint32_t>(item_src[s] + tile_rel) * ES;
            if constexpr (LM == LOAD_PAIR32) {
                // A pair is one 4-byte load (2-byte aligned in the odd rows of a plane of odd width). The last column of such
                // a plane has no right neighbour in its row, and at the very end of the tensor none at all: it is fetched
                // as the upper half of the pair that starts one column to its left. (Planes of even width never meet this
                // case; confining the extra instructions per item to odd widths behind uniform branches measured slower
                // on every layer.)
                off0[s] = ok0 ? (ok1 ? src : src - ES) : 0u;
            } else {
                off0[s] = ok0 ? src : 0u;
            }
            off1[s] = ok1 ? src + ES : 0u;
            z0 |= ok0 ? 0u : (1u << s);
            z1 |= ok1 ? 0u : (1u << s);
        }
        pre_zero0 = z0;
        pre_zero1 = z1;
        // A load address is a uniform base (timestep, image, chunk) plus a 32-bit lane offset that walks the 8 channels of
        // the group: one vector add per load. Fewer than 8 input channels in all: the absent ones re-read the last real
        // one (their weights are 0).
        const uint32_t chan_stride = static_cast<uint32_t>(plane) * ES;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            const char* __restrict__ base = reinterpret_cast<const char*>(static_cast<const XT*>(kernarg_table_entry(0, t)) + origin);
#pragma unroll
            for (int s = 0; s < SS; ++s) {
                if (item_cg[s] >= 0) {
                    uint32_t v0 = off0[s], v1 = off1[s];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        if constexpr (LM == LOAD_PAIR32) {
                            pre[s][t][j][0] = *reinterpret_cast<const uint32_t*>(base + v0);
                        } else if constexpr (LM == LOAD_2X16) {
                            pre[s][t][j][0] = *reinterpret_cast<const uint16_t*>(base + v0);
                            pre[s][t][j][1] = *reinterpret_cast<const uint16_t*>(base + v1);
                        } else {
                            pre[s][t][j][0] = *reinterpret_cast<const uint32_t*>(base + v0);
                            pre[s][t][j][1] = *reinterpret_cast<const uint32_t*>(base + v1);
                        }
                        const uint32_t step = j < last_channel ? chan_stride : 0u;   // uniform
                        v0 += step;
                        v1 += step;
                    }
                }
            }
        }
    };

    // Registers -> LDS, transposed to [pixel][channel]; padding and absent channels become zeros.
    auto write_lds = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            if (item_cg[s] >= 0) {
                const bool zero0 = (pre_zero0 >> s) & 1u, zero1 = (pre_zero1 >> s) & 1u;
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    cv_u32x4 lo, hi;
                    if constexpr (LM == LOAD_2XF32) {
                        // fp32: the high terms to the item's place, the low terms lo_off bytes behind them.
                        cv_u32x4 lo2, hi2;
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const float a0 = __uint_as_float(pre[s][t][2 * k][0]), a1 = __uint_as_float(pre[s][t][2 * k + 1][0]);
                            const float b0 = __uint_as_float(pre[s][t][2 * k][1]), b1 = __uint_as_float(pre[s][t][2 * k + 1][1]);
                            lo[k] = split_bf16_bits(a0, false) | (split_bf16_bits(a1, false) << 16);
                            hi[k] = split_bf16_bits(b0, false) | (split_bf16_bits(b1, false) << 16);
                            lo2[k] = zero0 ? 0u : (split_bf16_bits(a0, true) | (split_bf16_bits(a1, true) << 16));
                            hi2[k] = zero1 ? 0u : (split_bf16_bits(b0, true) | (split_bf16_bits(b1, true) << 16));
                        }
                        unsigned char* dst2 = lds + t * tile_bytes + item_dst[s] + lo_off;
                        *reinterpret_cast<cv_u32x4*>(dst2) = lo2;
                        *reinterpret_cast<cv_u32x4*>(dst2 + g.pitch) = hi2;
                        // (a low term is +0 or -0 when the value is exact in bf16: the sign bits do not count)
                        if (((lo2[0] | lo2[1] | lo2[2] | lo2[3] | hi2[0] | hi2[1] | hi2[2] | hi2[3]) & 0x7fff7fffu) != 0u) stage_has_low_terms = 1;
                    } else if constexpr (LM == LOAD_PAIR32) {
                        // An item whose first column is real and whose second is not is a row's last column: its first
                        // column sits in the upper halves.
                        const uint32_t first = (!zero0 && zero1) ? 0x07060302u : 0x05040100u;
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            lo[k] = __builtin_amdgcn_perm(pre[s][t][2 * k + 1][0], pre[s][t][2 * k][0], first);
                            hi[k] = __builtin_amdgcn_perm(pre[s][t][2 * k + 1][0], pre[s][t][2 * k][0], 0x07060302u);
                        }
                    } else {
                        uint32_t e0[8], e1[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            e0[j] = pre[s][t][j][0];
                            e1[j] = pre[s][t][j][1];
                        }
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            lo[k] = e0[2 * k] | (e0[2 * k + 1] << 16);
                            hi[k] = e1[2 * k] | (e1[2 * k + 1] << 16);
                        }
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        lo[k] = zero0 ? 0u : lo[k];
                        hi[k] = zero1 ? 0u : hi[k];
                    }
                    unsigned char* dst = lds + t * tile_bytes + item_dst[s];
                    *reinterpret_cast<cv_u32x4*>(dst) = lo;
                    *reinterpret_cast<cv_u32x4*>(dst + g.pitch) = hi;
                }
            }
        }
    };

    // ---- tile walk: an XCD takes a contiguous range of the pixel tiles (neighbouring tiles share halo pixels and, where a
    // tile row is shorter than a cache line, the lines they store to: both then meet in one L2); consecutive work items =
    // output-channel tiles (an XCD's L2 serves every activation tile to all of its output-channel tiles). Layers whose weights outweigh their
    // activations turn this around (oc_major): an XCD takes the output-channel tiles congruent to it for all pixel tiles, so
    // that its L2 holds an eighth of the weights instead of all of them.
    const int xcd = blockIdx.x & 7;
    const int slots_per_xcd = gridDim.x >> 3;
    const int n_px_tiles = g.img_groups * g.tiles_img;       // a tile spans TI images (TI > 1: whole output planes)
    const int oc_per_xcd = g.oc_major ? (g.oc_tiles >> 3) : g.oc_tiles;
    const int px_base = n_px_tiles >> 3, px_rem = n_px_tiles & 7;
    const int px_start = g.oc_major ? 0 : xcd * px_base + min(xcd, px_rem);
    const int work_per_xcd = (g.oc_major ? n_px_tiles : px_base + (xcd < px_rem ? 1 : 0)) * oc_per_xcd;
    int work = blockIdx.x >> 3;
    int oc_tile = 0, img = 0, oh0 = 0, ow0 = 0;
    auto decode = [&](int w, int& oc_t, int& n, int& r0, int& c0) __attribute__((always_inline)) -> bool {
        if (w >= work_per_xcd) return false;
        const int pt = fast_div(w, g.d_oc_tiles);
        const int px_tile = px_start + pt;
        if (px_tile >= n_px_tiles) return false;
        oc_t = g.oc_major ? (w - pt * oc_per_xcd) * 8 + xcd : w - pt * g.oc_tiles;
        const int group = fast_div(px_tile, g.d_tiles_img);
        const int in_img = px_tile - group * g.tiles_img;
        n = group * g.TI;
        const int ty = fast_div(in_img, g.d_tiles_x);
        r0 = ty * g.TH;
        c0 = (in_img - ty * g.tiles_x) * g.TW;
        return true;
    };
    auto halo_origin = [&](int r0, int c0, int& ih_lo, int& iw_lo) __attribute__((always_inline)) {
        ih_lo = r0 * g.sh - g.ph;
        iw_lo = c0 * g.sw - g.pw;
        if (pair_shift && (iw_lo & 1)) iw_lo -= 1;
    };
    bool have_tile = decode(work, oc_tile, img, oh0, ow0);
    if (have_tile) {
        int ih_lo, iw_lo;
        halo_origin(oh0, ow0, ih_lo, iw_lo);
        issue_loads(0, img, ih_lo, iw_lo);
        fetch_bias(oc_tile);
    }

    // ---- kernel constants of the matrix loop: this lane's pixel (block pixel wm * 32 + l32) inside the halo tile.
    const int mpix = wm * 32 + l32;
    const int mpi = fast_div(mpix, g.d_tile_px);             // image of the tile
    const int mrem = mpix - mpi * tile_px;
    const int mpr = fast_div(mrem, g.d_TW);
    const int mpc = mrem - mpr * g.TW;
    const bool m_inside = mpi < g.TI;                        // lanes beyond the tile read pixel (0, 0): finite, never stored
    const uint32_t b_base = static_cast<uint32_t>(m_inside ? ((mpi * g.NR + mpr * g.sh) * g.WT + mpc * g.sw) * g.pitch : 0);

    // ---- kernel constants of the epilogue: lane = (channel row lane >> 2 of 16, pixels 8 (lane & 3) .. + 7 of the wave's 32).
    const int row16 = lane >> 2;
    const int pcx = lane & 3;
    const int epix = wm * 32 + pcx * 8;
    const int epi = fast_div(epix, g.d_tile_px);
    const int erem = epix - epi * tile_px;
    const int epr = fast_div(erem, g.d_TW);
    const int epc = erem - epr * g.TW;
    const bool lo_inside = epix + 4 <= g.TI * tile_px;       // FAST: planes and tiles are multiples of 4 (8 with 16-byte runs), so
    const bool hi_inside = epix + 8 <= g.TI * tile_px;       // each half of a lane's run of 8 pixels is inside or outside as a whole
    const uint32_t image_out = static_cast<uint32_t>(g.Cout) * static_cast<uint32_t>(g.Ho * g.Wo);
    const uint32_t lane_px = static_cast<uint32_t>(epi) * image_out + static_cast<uint32_t>(epr * g.Wo + epc);
    // The second half of the lane's run of 8 (pixels epix + 4 .. + 7): contiguous with the first half inside an image, but
    // with tiles of several whole planes of 4 pixels (2x2 planes) it lies in the next image of the tile.
    const int epi_hi = fast_div(epix + 4, g.d_tile_px);
    const int erem_hi = epix + 4 - epi_hi * tile_px;
    const int epr_hi = fast_div(erem_hi, g.d_TW);
    const uint32_t lane_px_hi = static_cast<uint32_t>(epi_hi) * image_out + static_cast<uint32_t>(epr_hi * g.Wo + (erem_hi - epr_hi * g.TW));
    float* __restrict__ stage_wr = stage + (half * 4) * kMmStagePitch + l32;
    const float* __restrict__ stage_rd = stage + row16 * kMmStagePitch + pcx * 8;
    const float c0f = lif.charge_mode == CHARGE_IF ? 0.0f : 1.0f;
    const float c1f = lif.charge_mode == CHARGE_IF ? 1.0f : lif.inv_tau;
    const bool divide = lif.charge_mode == CHARGE_DIVIDE;   // tau is not a power of two: a true division

    while (have_tile) {
        int ih_lo, iw_lo;
        halo_origin(oh0, ow0, ih_lo, iw_lo);
        // Column of the tile's first output pixel inside the halo tile (0, or 1 when the halo start was aligned down).
        const int col0 = (ow0 * g.sw - g.pw) - iw_lo;
        const int ocf0 = ((oc_tile << g.wn_log2) + wn) * 2;
        const bool wave_has_work = ocf0 < nocf;
        const uint16_t* __restrict__ wlane = wpacked + lane * 8;
        const int64_t w_off0 = static_cast<int64_t>(min(ocf0, nocf - 1)) * frag_stride_ocf;
        const int64_t w_off1 = static_cast<int64_t>(min(ocf0 + 1, nocf - 1)) * frag_stride_ocf;

        cv_f32x16 acc[TT][2];
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[t][f][r] = 0.0f;

        int next_work = work, next_oc_tile = oc_tile, next_img = img, next_oh0 = oh0, next_ow0 = ow0;
        bool next_tile = false;
        int stage_now = 0;       // the LDS stage the matrix steps are working on
        // One pair of k-slots: slot 2 * pair + half -> (tap, channel group); both halves' LDS offsets are computed on the
        // scalar unit, a lane picks its half's.
        auto mma_pair = [&](int q, const unsigned char* __restrict__ bp0, const cv_u32x4& a0, const cv_u32x4& a1) __attribute__((always_inline)) {
            if constexpr (PARTS > 1) {   // q counts the stage's pairs three times over: part 2 reads the low terms
                const int sp = min(g.stage_chunks, g.nchunks_r - stage_now * g.stage_chunks) * g.npairs;
                const int part = q >= 2 * sp ? 2 : (q >= sp ? 1 : 0);
                q -= part * sp;
                bp0 += part == 2 ? lo_off : 0;
            }
            const int sub = fast_div(q, g.d_npairs);                 // chunk inside the stage
            const int pair = q - sub * g.npairs;
            const unsigned char* __restrict__ bp = bp0 + sub * (groups * 16);
            const int s0 = 2 * pair, s1 = 2 * pair + 1;
            // With a single channel group an odd tap count leaves the last k-slot empty (zero weights): it re-reads the last tap.
            const int tap0 = s0 >> g.groups_log2, tap1 = min(s1 >> g.groups_log2, taps - 1);
            const int kh0 = fast_div(tap0, g.d_KW), kh1 = fast_div(tap1, g.d_KW);
            const int off_even = ((kh0 * g.WT) + (tap0 - kh0 * g.KW)) * g.pitch + (s0 & (groups - 1)) * 16;
            const int off_odd = ((kh1 * g.WT) + (tap1 - kh1 * g.KW)) * g.pitch + (s1 & (groups - 1)) * 16;
            const unsigned char* __restrict__ bq = bp + (half ? off_odd : off_even);
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                const cv_u32x4 b = *reinterpret_cast<const cv_u32x4*>(bq + t * tile_bytes);
                acc[t][0] = cv_mfma<F16>(a0, b, acc[t][0]);
                acc[t][1] = cv_mfma<F16>(a1, b, acc[t][1]);
            }
        };
        // Weight fragments stream from L2 two pairs ahead of their use, through three register sets.
        // `gpair`: first pair of the stage + the pair's index in the stage (fp32: the index runs over the three parts, each
        // of which lies nchunks_r chunks further in the packed weight).
        auto load_frags = [&](int gpair, cv_u32x4& a0, cv_u32x4& a1) __attribute__((always_inline)) {
            if constexpr (PARTS > 1) {
                const int first = stage_now * g.stage_chunks * g.npairs;
                const int sp = min(g.stage_chunks, g.nchunks_r - stage_now * g.stage_chunks) * g.npairs;
                const int q = gpair - first;
                const int part = q >= 2 * sp ? 2 : (q >= sp ? 1 : 0);
                gpair += part * (g.nchunks_r * g.npairs - sp);
            }
            const int64_t o = static_cast<int64_t>(min(gpair, total_pairs - 1)) * (kFragBytes / 2);
            a0 = *reinterpret_cast<const cv_u32x4*>(wlane + w_off0 + o);
            a1 = *reinterpret_cast<const cv_u32x4*>(wlane + w_off1 + o);
        };
        cv_u32x4 wa[3][2];
        for (int chunk = 0; chunk < nstages; ++chunk) {        // `chunk` counts LDS stages from here on
            stage_now = chunk;
            const int gp0 = chunk * g.stage_chunks * g.npairs;
            const int spairs_all = PARTS * min(g.stage_chunks, g.nchunks_r - chunk * g.stage_chunks) * g.npairs;   // pairs of this stage (all parts)
            load_frags(gp0 + wk, wa[0][0], wa[0][1]);  // in flight across the barriers and the LDS writes below
            load_frags(gp0 + wk + WK, wa[1][0], wa[1][1]);
            if constexpr (PARTS > 1) {
                if (tid == 0) stage_has_low_terms = 0;     // every wave has read the previous stage's flag before it got here
            }
            __syncthreads();   // every wave is done reading the previous stage (and with the previous tile's epilogue)
            write_lds();       // waits for the stage's loads
            if (chunk == 0 && tid < (64 << g.wn_log2)) bias_lds[tid] = bias_pre;
            __syncthreads();
            int spairs = spairs_all;
            if constexpr (PARTS > 1) {
                if (__builtin_amdgcn_readfirstlane(static_cast<int>(stage_has_low_terms)) == 0) spairs = (spairs_all / PARTS) * 2;
            }
            // ---- the stage after this one: next chunk, or the first chunk of the next tile.
            {
                int nc = chunk + 1, nimg = img, nih = ih_lo, niw = iw_lo;
                bool more = true;
                if (nc == nstages) {
                    nc = 0;
                    next_work = work + slots_per_xcd;
                    next_tile = decode(next_work, next_oc_tile, next_img, next_oh0, next_ow0);
                    more = next_tile && !SK;   // split K: the next tile's loads go out after the epilogue (registers)
                    nimg = next_img;
                    halo_origin(next_oh0, next_ow0, nih, niw);
                }
                if (more) {
                    issue_loads(nc, nimg, nih, niw);
                    if (nc == 0) fetch_bias(next_oc_tile);
                }
            }
            if (wave_has_work) {
                const unsigned char* __restrict__ bp = lds + b_base + static_cast<uint32_t>(col0 * g.pitch);
                // This wave's pairs of the chunk: wk, wk + WK, ... (every pair when K is not split).
                for (int pair = wk; pair < spairs; pair += 3 * WK) {
                    load_frags(gp0 + pair + 2 * WK, wa[2][0], wa[2][1]);
                    mma_pair(pair, bp, wa[0][0], wa[0][1]);
                    if (pair + WK < spairs) {
                        load_frags(gp0 + pair + 3 * WK, wa[0][0], wa[0][1]);
                        mma_pair(pair + WK, bp, wa[1][0], wa[1][1]);
                    }
                    if (pair + 2 * WK < spairs) {
                        load_frags(gp0 + pair + 4 * WK, wa[1][0], wa[1][1]);
                        mma_pair(pair + 2 * WK, bp, wa[2][0], wa[2][1]);
                    }
                }
            }
        }

        // ---- epilogue. h = v + (x - v * c0) * c1 covers tau <= 1 and power-of-two tau exactly.
        // FAST: 16 channel rows x 32 pixels at a time go through the wave's LDS stage, so that a lane owns 8 consecutive pixels
        // of one channel row (16- or 8-byte accesses); the membrane of those 8 neurons lives in registers across the TT steps.
        // General variant: straight from the accumulator layout - a lane owns ONE pixel and 8 channel rows per group, the 32
        // lanes of a half-wave store 32 consecutive pixels of a row (coalesced 2-byte spike stores whatever the alignment of
        // the planes), one validity bit per lane instead of one per element.
        const bool vf32 = FAST || g.v_is_f32;
        const bool wide = !FAST || g.run8 == 8;          // FAST: 16-byte spike accesses, or 8-byte ones when runs are only 8-byte aligned
        const uint32_t okmask = FAST ? ((lo_inside ? 0x0fu : 0u) | (hi_inside ? 0xf0u : 0u))
                                     : ((m_inside && img + mpi < g.N && oh0 + mpr < g.Ho && ow0 + mpc < g.Wo) ? 0xffu : 0u);
        // Element offset of the lane's first pixel (FAST: of its run of 8) from the tile origin of its channel row.
        const uint32_t px0 = FAST ? lane_px : static_cast<uint32_t>(mpi) * image_out + static_cast<uint32_t>(mpr * g.Wo + mpc);
        const uint32_t px4 = lane_px_hi;   // FAST: offset of the run's second half
        const int64_t tile_off = static_cast<int64_t>(img) * g.Cout * po + oh0 * g.Wo + ow0;   // uniform, elements
        const bool analog = g.analog_out != 0;   // neuron-free output: conv + bias (+ residual) where the spikes would go

        // One group = 8 accumulator registers of a 32-row fragment: FAST, after the transposition, this lane's channel row
        // row16 of the group's 16 rows; general variant, the lane's 8 rows first + {0..3, 8..11} with
        // first = 32 fragment + 16 (gidx & 1) + 4 half. `row_ok`: the lane has anything to load or store in the group.
        auto first_row = [&](int gidx) __attribute__((always_inline)) -> int {
            return (ocf0 + (gidx >> 1)) * 32 + (gidx & 1) * 16 + (FAST ? row16 : 4 * half);
        };
        auto row_delta = [&](int rr) __attribute__((always_inline)) -> int { return 8 * (rr >> 2) + (rr & 3); };
        // General variant: all 16 channel rows of the group exist (uniform; true for every group when Cout % 16 == 0), so
        // the per-row checks and their branches drop out.
        auto group_full = [&](int gidx) __attribute__((always_inline)) -> bool {
            return (ocf0 + (gidx >> 1)) * 32 + (gidx & 1) * 16 + 16 <= g.Cout;
        };
        auto group_row = [&](int gidx, bool& row_ok, uint32_t& row_off, float (&bvv)[8]) __attribute__((always_inline)) {
            const int oc = first_row(gidx);
            row_ok = wave_has_work && (FAST || oc < g.Cout) && okmask != 0;
            row_off = static_cast<uint32_t>(min(oc, g.Cout - 1)) * static_cast<uint32_t>(po);
            if constexpr (FAST) {
                bvv[0] = bias_lds[oc - (oc_tile << g.wn_log2) * 64];
            } else {   // rows beyond Cout hold zeros
#pragma unroll
                for (int rr = 0; rr < 8; ++rr) bvv[rr] = bias_lds[oc - (oc_tile << g.wn_log2) * 64 + row_delta(rr)];
            }
        };
        auto load_membrane = [&](int gidx, bool row_ok, uint32_t row_off, float (&v)[8]) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = 0.0f;
            if (v_init == nullptr || !row_ok) return;
            if constexpr (FAST) {
                const float* src = static_cast<const float*>(v_init) + tile_off + row_off + px0;
                if (okmask & 0x0fu) {
                    const Pack<float, 4> lo = *reinterpret_cast<const Pack<float, 4>*>(src);
#pragma unroll
                    for (int k = 0; k < 4; ++k) v[k] = lo.v[k];
                }
                if (okmask & 0xf0u) {
                    const Pack<float, 4> hi = *reinterpret_cast<const Pack<float, 4>*>(src - px0 + px4);
#pragma unroll
                    for (int k = 0; k < 4; ++k) v[4 + k] = hi.v[k];
                }
            } else {
                const int oc = first_row(gidx);
                const bool all_rows = group_full(gidx);
#pragma unroll
                for (int rr = 0; rr < 8; ++rr) {
                    if (all_rows || oc + row_delta(rr) < g.Cout) {
                        const int64_t at = tile_off + row_off + static_cast<uint32_t>(row_delta(rr) * po) + px0;
                        v[rr] = vf32 ? static_cast<const float*>(v_init)[at] : to_float(static_cast<const XT*>(v_init)[at]);
                    }
                }
            }
        };
        auto store_membrane = [&](int gidx, bool row_ok, uint32_t row_off, const float (&v)[8]) __attribute__((always_inline)) {
            if (!row_ok || analog) return;
            if constexpr (FAST) {
                float* dst = static_cast<float*>(v_out) + tile_off + row_off + px0;
                Pack<float, 4> lo, hi;
#pragma unroll
                for (int k = 0; k < 4; ++k) { lo.v[k] = v[k]; hi.v[k] = v[4 + k]; }
                if (okmask & 0x0fu) *reinterpret_cast<Pack<float, 4>*>(dst) = lo;
                if (okmask & 0xf0u) *reinterpret_cast<Pack<float, 4>*>(dst - px0 + px4) = hi;
            } else {
                const int oc = first_row(gidx);
                if (group_full(gidx)) {
                    if (vf32) {
                        float* __restrict__ dst = static_cast<float*>(v_out) + tile_off + row_off;
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) dst[static_cast<uint32_t>(row_delta(rr) * po) + px0] = v[rr];
                    } else {
                        XT* __restrict__ dst = static_cast<XT*>(v_out) + tile_off + row_off;
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) dst[static_cast<uint32_t>(row_delta(rr) * po) + px0] = from_float<XT>(v[rr]);
                    }
                    return;
                }
#pragma unroll
                for (int rr = 0; rr < 8; ++rr) {
                    if (oc + row_delta(rr) < g.Cout) {
                        const int64_t at = tile_off + row_off + static_cast<uint32_t>(row_delta(rr) * po) + px0;
                        if (vf32) static_cast<float*>(v_out)[at] = v[rr];
                        else static_cast<XT*>(v_out)[at] = from_float<XT>(v[rr]);
                    }
                }
            }
        };
        // The neuron (or, in the neuron-free mode, the conversion of the sum) of one element.
        auto neuron = [&](float x, float& v) __attribute__((always_inline)) -> XT {
            bool fired;
            if constexpr (FAST) {   // the common neuron: power-of-two tau, hard reset
                const float h = v + (x - v) * lif.inv_tau;
                fired = h >= lif.v_threshold;
                v = fired ? lif.v_reset : h;
            } else {
                const float h = divide ? v + __fdiv_rn(x - v, lif.tau) : v + (x - v * c0f) * c1f;
                fired = h >= lif.v_threshold;
                v = fired ? (lif.soft_reset ? h - lif.v_threshold : lif.v_reset) : h;
            }
            return spike_value<XT>(fired);
        };
        // One LIF step of a group: the lane's 8 sums arrive in accumulator layout (xin = rows 8 (gidx & 1) .. + 7 of its
        // 32-row fragment, for its pixel). FAST: transposed through the wave's stage, then bias (+ residual), LIF, one wide
        // spike store. General variant: bias (+ residual), LIF and a 2-byte store per row, in place.
        auto lif_step_group = [&](int t, int gidx, bool row_ok, uint32_t row_off, const float (&bvv)[8], const float (&xin)[8], float (&v)[8]) __attribute__((always_inline)) {
            XT* __restrict__ out_t = spikes + t * g.spike_step_stride + tile_off + row_off;
            const XT* __restrict__ res_t = nullptr;
            if (has_residual) res_t = static_cast<const XT*>(kernarg_table_entry(sizeof(StepPtrs), t)) + tile_off + row_off;
            if constexpr (FAST) {
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int rr = 0; rr < 8; ++rr) stage_wr[((rr >> 2) * 8 + (rr & 3)) * kMmStagePitch] = xin[rr];
                __builtin_amdgcn_wave_barrier();
                const cv_f32x4 xlo = *reinterpret_cast<const cv_f32x4*>(stage_rd);
                const cv_f32x4 xhi = *reinterpret_cast<const cv_f32x4*>(stage_rd + 4);
                float x[8];
#pragma unroll
                for (int k = 0; k < 4; ++k) { x[k] = xlo[k] + bvv[0]; x[4 + k] = xhi[k] + bvv[0]; }
                if (has_residual && row_ok) {
                    if (wide) {
                        const Pack<XT, 8> rr8 = *reinterpret_cast<const Pack<XT, 8>*>(res_t + px0);
#pragma unroll
                        for (int k = 0; k < 8; ++k) x[k] += to_float(rr8.v[k]);
                    } else {
                        if (okmask & 0x0fu) {
                            const Pack<XT, 4> ra = *reinterpret_cast<const Pack<XT, 4>*>(res_t + px0);
#pragma unroll
                            for (int k = 0; k < 4; ++k) x[k] += to_float(ra.v[k]);
                        }
                        if (okmask & 0xf0u) {
                            const Pack<XT, 4> rb = *reinterpret_cast<const Pack<XT, 4>*>(res_t + px4);
#pragma unroll
                            for (int k = 0; k < 4; ++k) x[4 + k] += to_float(rb.v[k]);
                        }
                    }
                }
                Pack<XT, 8> sp;
                if (analog) {   // uniform: no neuron, the sums themselves go out
#pragma unroll
                    for (int k = 0; k < 8; ++k) sp.v[k] = from_float<XT>(x[k]);
                } else {
#pragma unroll
                    for (int k = 0; k < 8; ++k) sp.v[k] = neuron(x[k], v[k]);
                }
                if (row_ok) {
                    if (wide) {
                        *reinterpret_cast<Pack<XT, 8>*>(out_t + px0) = sp;
                    } else {
                        Pack<XT, 4> sa, sb;
#pragma unroll
                        for (int k = 0; k < 4; ++k) { sa.v[k] = sp.v[k]; sb.v[k] = sp.v[4 + k]; }
                        if (okmask & 0x0fu) *reinterpret_cast<Pack<XT, 4>*>(out_t + px0) = sa;
                        if (okmask & 0xf0u) *reinterpret_cast<Pack<XT, 4>*>(out_t + px4) = sb;
                    }
                }
            } else {
                if (!row_ok) return;
                const int oc = first_row(gidx);
                if (group_full(gidx)) {
                    float x[8];
#pragma unroll
                    for (int rr = 0; rr < 8; ++rr) x[rr] = xin[rr] + bvv[rr];
                    if (has_residual) {
                        XT res[8];
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) res[rr] = res_t[static_cast<uint32_t>(row_delta(rr) * po) + px0];
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) x[rr] += to_float(res[rr]);
                    }
                    if (analog) {
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) out_t[static_cast<uint32_t>(row_delta(rr) * po) + px0] = from_float<XT>(x[rr]);
                    } else {
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) out_t[static_cast<uint32_t>(row_delta(rr) * po) + px0] = neuron(x[rr], v[rr]);
                    }
                    return;
                }
#pragma unroll
                for (int rr = 0; rr < 8; ++rr) {
                    if (oc + row_delta(rr) < g.Cout) {
                        const uint32_t at = static_cast<uint32_t>(row_delta(rr) * po) + px0;
                        float x = xin[rr] + bvv[rr];
                        if (has_residual) x += to_float(res_t[at]);
                        out_t[at] = analog ? from_float<XT>(x) : neuron(x, v[rr]);
                    }
                }
            }
        };

        if constexpr (!SK) {
            if (wave_has_work) {
#pragma unroll
                for (int gidx = 0; gidx < 4; ++gidx) {
                    bool row_ok;
                    uint32_t row_off;
                    float bvv[8], v[8];
                    group_row(gidx, row_ok, row_off, bvv);
                    load_membrane(gidx, row_ok, row_off, v);
                    if constexpr (TT == 1) {
                        // One stage of input: a single timestep, or one analog frame that feeds all g.T timesteps.
                        float xin[8];
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr) xin[rr] = acc[0][gidx >> 1][(gidx & 1) * 8 + rr];
                        for (int t = 0; t < g.T; ++t) lif_step_group(t, gidx, row_ok, row_off, bvv, xin, v);
                    } else {
#pragma unroll
                        for (int t = 0; t < TT; ++t) {
                            if (t < g.T) {
                                float xin[8];
#pragma unroll
                                for (int rr = 0; rr < 8; ++rr) xin[rr] = acc[t][gidx >> 1][(gidx & 1) * 8 + rr];
                                lif_step_group(t, gidx, row_ok, row_off, bvv, xin, v);
                            }
                        }
                    }
                    store_membrane(gidx, row_ok, row_off, v);
                }
            }
        } else {
            // Split K: the WK waves that share an output tile add their partial sums through LDS, one timestep per round (the
            // halo tiles are dead by then). A group has one owner wave, which adds the WK partial sums in a fixed order and
            // runs that step's LIF right away, so only the membranes stay in registers between rounds.
            float* __restrict__ part = reinterpret_cast<float*>(lds);      // [tile wave][wk][quad 0..7][lane][4]
            const int wt = wave & ((1 << (g.wm_log2 + g.wn_log2)) - 1);
            bool row_ok[2];
            uint32_t row_off[2];
            float bvv[2][8], v[2][8];
#pragma unroll
            for (int gidx = 0; gidx < 4; ++gidx) {
                const int owner = g.wk_log2 == 1 ? (gidx >> 1) : (gidx << (g.wk_log2 - 2));
                if (owner == wk) {
                    group_row(gidx, row_ok[gidx & 1], row_off[gidx & 1], bvv[gidx & 1]);
                    load_membrane(gidx, row_ok[gidx & 1], row_off[gidx & 1], v[gidx & 1]);
                }
            }
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                if (t < g.T) {   // uniform: every wave takes the same rounds
                    __syncthreads();   // previous round read; first round: every wave is done with the halo tiles
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const cv_f32x4 four = {acc[t][f][4 * q], acc[t][f][4 * q + 1], acc[t][f][4 * q + 2], acc[t][f][4 * q + 3]};
                            *reinterpret_cast<cv_f32x4*>(part + (((wt * WK + wk) * 8 + f * 4 + q) * 64 + lane) * 4) = four;
                        }
                    __syncthreads();
#pragma unroll
                    for (int gidx = 0; gidx < 4; ++gidx) {
                        const int owner = g.wk_log2 == 1 ? (gidx >> 1) : (gidx << (g.wk_log2 - 2));
                        if (owner == wk) {
                            cv_f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
                            for (int k = 0; k < WK; ++k) {
                                const float* __restrict__ src = part + (((wt * WK + k) * 8 + gidx * 2) * 64 + lane) * 4;
                                lo += *reinterpret_cast<const cv_f32x4*>(src);
                                hi += *reinterpret_cast<const cv_f32x4*>(src + 256);
                            }
                            float xin[8];
#pragma unroll
                            for (int k = 0; k < 4; ++k) { xin[k] = lo[k]; xin[4 + k] = hi[k]; }
                            if constexpr (TT == 1) {   // one stage of input feeds all g.T timesteps
                                for (int ts = 0; ts < g.T; ++ts)
                                    lif_step_group(ts, gidx, row_ok[gidx & 1], row_off[gidx & 1], bvv[gidx & 1], xin, v[gidx & 1]);
                            } else {
                                lif_step_group(t, gidx, row_ok[gidx & 1], row_off[gidx & 1], bvv[gidx & 1], xin, v[gidx & 1]);
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int gidx = 0; gidx < 4; ++gidx) {
                const int owner = g.wk_log2 == 1 ? (gidx >> 1) : (gidx << (g.wk_log2 - 2));
                if (owner == wk) store_membrane(gidx, row_ok[gidx & 1], row_off[gidx & 1], v[gidx & 1]);
            }
        }
        if (SK && next_tile) {
            int nih, niw;
            halo_origin(next_oh0, next_ow0, nih, niw);
            issue_loads(0, next_img, nih, niw);
            fetch_bias(next_oc_tile);
        }
        work = next_work;
        oc_tile = next_oc_tile;
        img = next_img;
        oh0 = next_oh0;
        ow0 = next_ow0;
        have_tile = next_tile;
    }
}

template <typename XT, int TT, int NW>
int launch_conv_mm_tt(const ConvLaunch& L, int load_mode, bool fast) {
    const bool split_k = L.g.wk_log2 > 0;
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), NW * 64, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.has_residual, L.g, L.wpacked, L.bias, L.v_init,
                                                                    static_cast<XT*>(L.spikes), L.v_out, L.lif);
        return check_launch("snnf_conv_lif");
    };
    auto pick = [&](auto lm) -> int {
        constexpr int LMV = decltype(lm)::value;
        if constexpr (NW == 8) {
            if (split_k)
                return fast ? run(conv_mm_lif_kernel<XT, TT, LMV, true, true, 8>) : run(conv_mm_lif_kernel<XT, TT, LMV, false, true, 8>);
            return fast ? run(conv_mm_lif_kernel<XT, TT, LMV, true, false, 8>) : run(conv_mm_lif_kernel<XT, TT, LMV, false, false, 8>);
        } else {   // half-size workgroups exist in the fast variant only
            if (!fast) return fail(SNNF_ERR_LAUNCH, "snnf_conv_lif: no general variant with %d waves", NW);
            return split_k ? run(conv_mm_lif_kernel<XT, TT, LMV, true, true, NW>) : run(conv_mm_lif_kernel<XT, TT, LMV, true, false, NW>);
        }
    };
    if constexpr (sizeof(XT) == 4) {
        return pick(std::integral_constant<int, LOAD_2XF32>{});
    } else {
        if (load_mode == LOAD_PAIR32) return pick(std::integral_constant<int, LOAD_PAIR32>{});
        return pick(std::integral_constant<int, LOAD_2X16>{});
    }
}

template <typename XT, int NW = 8>
int launch_conv_mm(const ConvLaunch& L, int tt, int load_mode, bool fast) {
    if (tt == 4) return launch_conv_mm_tt<XT, 4, NW>(L, load_mode, fast);
    if (tt == 2) return launch_conv_mm_tt<XT, 2, NW>(L, load_mode, fast);
    return launch_conv_mm_tt<XT, 1, NW>(L, load_mode, fast);
}

}  // namespace snnf
