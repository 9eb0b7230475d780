// Time-outer variant of the implicit-GEMM conv+LIF kernel, for layers bound by HBM bandwidth rather than by the
// matrix cores (pointwise convolutions, few input channels, analog frames shared by all timesteps).
//
// Same operand mapping as snnf_conv_kernel.h (M = output channels, N = output pixels), but a wave owns 32 channels x 64
// pixels and one timestep is accumulated at a time: only 32 accumulator registers per lane, the fp32 membrane of the
// lane's 32 neurons stays in registers across ALL T steps (any T, it never touches HBM between steps), and the LDS
// tile holds a single timestep. The small footprint lets two workgroups share a CU, so one workgroup's loads, matrix
// work and LIF/stores overlap the other's. Per step the accumulators are transposed through a wave-private LDS stage
// (no workgroup barrier) so that a lane owns 8 consecutive pixels of one channel row and spikes leave as 16-byte
// stores. A frame shared by all timesteps is convolved once and only the LIF recurrence is repeated.
#pragma once

#include "snnf_conv_kernel.h"

namespace snnf {

constexpr int kToutStagePitch = 12;                                           // floats per pixel of the stage (8 rows + padding)
constexpr int kToutStageFloats = 64 * kToutStagePitch;                        // per wave: 64 pixels x 8 channel rows
static_assert(4 * kToutStageFloats * sizeof(float) == kToutStageBytes, "planner and kernel disagree on the stage size");
__host__ __device__ constexpr int tout_staging_items(int load_mode) { return load_mode == LOAD_PAIR32 ? 4 : 2; }
constexpr int kToutNOF = 1;   // output-channel fragments per wave: 32 channels x 64 pixels keeps two to three workgroups per CU

// Entry `i` of a by-value pointer table, picked with a chain of scalar selects (a dynamically indexed kernel argument
// would be copied to scratch memory).
__device__ __forceinline__ const void* step_pointer(const StepPtrs& table, int i) {
    const void* p = table.p[0];
#pragma unroll
    for (int k = 1; k < SNNF_MAX_T_PER_LAUNCH; ++k) p = (i == k) ? table.p[k] : p;
    return p;
}

// STD: the common neuron (power-of-two tau, hard reset) with a shorter instruction sequence; otherwise the generic one.
template <typename XT, int LM, bool STD>
__global__ __launch_bounds__(kConvThreads, 2) void conv_lif_tout_kernel(const StepPtrs xs, const StepPtrs residuals,
                                                                        const int has_residual, const ConvGeom g,
                                                                        const uint16_t* __restrict__ wpacked,
                                                                        const float* __restrict__ bias,
                                                                        const void* __restrict__ v_init,
                                                                        XT* __restrict__ spikes,
                                                                        void* __restrict__ v_out, const LifParams lif) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    constexpr int RPE = LM == LOAD_PAIR32 ? 1 : 2;
    constexpr int SS = tout_staging_items(LM);   // staging slots per thread and chunk (one timestep at a time)
    constexpr int ES = static_cast<int>(sizeof(XT));
    constexpr int NOF = kToutNOF;
    constexpr int NG = NOF * 4;                   // epilogue row groups (8 channel rows each) per wave
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int wm = wave & ((1 << g.wm_log2) - 1);
    const int wn = wave >> g.wm_log2;

    const int groups = 1 << g.groups_log2;
    const int tile_bytes = g.NR * g.WT * g.pitch;
    const int zero_off = tile_bytes;
    float* __restrict__ stage = reinterpret_cast<float*>(lds + tile_bytes + g.pitch) + wave * kToutStageFloats;
    // Optional LDS copy of this workgroup's weight fragments: [wave column wn][fragment f][pair][lane] x 16 bytes.
    const unsigned char* __restrict__ wlds = lds + tile_bytes + g.pitch + kToutStageBytes;
    int loaded_oc_tile = -1;
    const int total_rows = g.N * g.Ho;
    const int64_t plane = static_cast<int64_t>(g.H) * g.W;
    const int po = g.Ho * g.Wo;
    const int WTP = g.WT >> 1;
    const bool pair_shift = LM == LOAD_PAIR32;
    const int nocf = (g.Cout + 31) >> 5;
    const int64_t frag_stride_ocf = static_cast<int64_t>(g.nchunks) * g.npairs * (kFragBytes / 2);
    const int total_pairs = g.nchunks * g.npairs;
    const int steps_with_input = g.shared_x ? 1 : g.T;

    if (tid < g.pitch / 4) reinterpret_cast<uint32_t*>(lds + zero_off)[tid] = 0u;

    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int slots_per_xcd = gridDim.x >> 3;
    const int n_px_tiles = g.tiles_x * g.tiles_y;
    const int px_per_xcd = (n_px_tiles + 7) >> 3;
    const int work_per_xcd = px_per_xcd * g.oc_tiles;

    uint32_t st_src[SS];
    uint32_t st_meta[SS];
    uint32_t pre[SS][8][RPE];

    auto compute_descriptors = [&](int px_tile) __attribute__((always_inline)) {
        const int tile_y = fast_div(px_tile, g.d_tiles_x);
        const int tile_x = px_tile - tile_y * g.tiles_x;
        const int q0 = tile_y * g.TH;
        const int q_last = min(q0 + g.TH, total_rows) - 1;
        const int n_first = fast_div(q0, g.d_Ho);
        const int g_lo = n_first * g.H + (q0 - n_first * g.Ho) * g.sh - g.ph;
        const int n_last = fast_div(q_last, g.d_Ho);
        const int rows = n_last * g.H + (q_last - n_last * g.Ho) * g.sh - g.ph + g.KH - g_lo;
        int iw_lo = tile_x * g.TW * g.sw - g.pw;
        if (pair_shift && (iw_lo & 1)) iw_lo -= 1;
        // Items are laid out for the tallest tile (NR input rows); a shorter tile leaves the items of its missing rows idle.
        const int stage_rows = g.NR * WTP;
        const int spatial_items = groups * stage_rows;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            const int e = s * kConvThreads + tid;
            int flags = 0, src = 0, dst = 0, cg = 0;
            if (e < spatial_items) {
                cg = fast_div(e, g.d_stage_rows);
                const int rem = e - cg * stage_rows;
                const int r = fast_div(rem, g.d_WTP);
                const int cp = rem - r * WTP;
                const int grow = g_lo + r;
                const int iw = iw_lo + cp * 2;
                dst = (r * g.WT + cp * 2) * g.pitch + cg * 16;
                if (r < rows && grow >= 0 && grow < g.N * g.H) {
                    const int xn = fast_div(grow, g.d_H);
                    const int ih = grow - xn * g.H;
                    src = max(0, ((xn * g.Cin + cg * 8) * g.H + ih) * g.W + iw + 1);
                    flags = 4 | ((iw >= 0 && iw < g.W) ? 1 : 0) | ((iw + 1 >= 0 && iw + 1 < g.W) ? 2 : 0);
                }
            }
            st_src[s] = static_cast<uint32_t>(src) * ES;
            st_meta[s] = static_cast<uint32_t>(dst) | (static_cast<uint32_t>(flags) << 20) | (static_cast<uint32_t>(cg) << 24);
        }
    };

    int pre_part = 0;       // fp32 tensors: which of the three parts of the channel axis `pre` holds (2: the low terms)
    auto issue_loads = [&](int step, int chunk) __attribute__((always_inline)) {
        if constexpr (LM == LOAD_2XF32) split_chunk(chunk, g.nchunks_r, pre_part, chunk);
        const char* __restrict__ base = static_cast<const char*>(step_pointer(xs, step)) + static_cast<int64_t>(chunk) * g.CK * plane * ES;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            const uint32_t flags = st_meta[s] >> 20;
            if (flags & 4) {
                const int nval = g.Cin - (chunk * g.CK + static_cast<int>((st_meta[s] >> 24) & 31u) * 8);
                const bool ok0 = flags & 1, ok1 = flags & 2;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const bool cok = j < nval;
                    const char* __restrict__ row = base + j * plane * ES;
                    if constexpr (LM == LOAD_PAIR32) {
                        pre[s][j][0] = (cok && ok0) ? *reinterpret_cast<const uint32_t*>(row + st_src[s] - 2) : 0u;
                    } else if constexpr (LM == LOAD_2X16) {
                        pre[s][j][0] = (cok && ok0) ? *reinterpret_cast<const uint16_t*>(row + st_src[s] - 2) : 0u;
                        pre[s][j][1] = (cok && ok1) ? *reinterpret_cast<const uint16_t*>(row + st_src[s]) : 0u;
                    } else {
                        pre[s][j][0] = (cok && ok0) ? *reinterpret_cast<const uint32_t*>(row + st_src[s] - 4) : 0u;
                        pre[s][j][1] = (cok && ok1) ? *reinterpret_cast<const uint32_t*>(row + st_src[s]) : 0u;
                    }
                }
            }
        }
    };

    auto write_lds = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            if ((st_meta[s] >> 20) & 4) {
                cv_u32x4 lo, hi;
                if constexpr (LM == LOAD_PAIR32) {
                    // dword j = (pixel 0, pixel 1) of channel j -> per pixel, channel pairs: one byte permute each.
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        lo[k] = __builtin_amdgcn_perm(pre[s][2 * k + 1][0], pre[s][2 * k][0], 0x05040100u);
                        hi[k] = __builtin_amdgcn_perm(pre[s][2 * k + 1][0], pre[s][2 * k][0], 0x07060302u);
                    }
                } else {
                    uint32_t e0[8], e1[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        if constexpr (LM == LOAD_2X16) {
                            e0[j] = pre[s][j][0];
                            e1[j] = pre[s][j][1];
                        } else {
                            e0[j] = split_bf16_bits(__uint_as_float(pre[s][j][0]), pre_part == 2);
                            e1[j] = split_bf16_bits(__uint_as_float(pre[s][j][1]), pre_part == 2);
                        }
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        lo[k] = e0[2 * k] | (e0[2 * k + 1] << 16);
                        hi[k] = e1[2 * k] | (e1[2 * k + 1] << 16);
                    }
                }
                unsigned char* dst = lds + (st_meta[s] & 0xfffffu);
                *reinterpret_cast<cv_u32x4*>(dst) = lo;
                *reinterpret_cast<cv_u32x4*>(dst + g.pitch) = hi;
            }
        }
    };

    int work = slot;
    auto px_tile_of = [&](int w) __attribute__((always_inline)) { return fast_div(w, g.d_oc_tiles) * 8 + xcd; };
    bool have_tile = work < work_per_xcd && px_tile_of(work) < n_px_tiles;
    if (have_tile) {
        compute_descriptors(px_tile_of(work));
        issue_loads(0, 0);
    }

    const int rg = lane >> 3;    // channel row of this lane inside a group of 8 (epilogue layout)
    const int pcx = lane & 7;    // pixel chunk: pixels 8 * pcx .. 8 * pcx + 7 of the wave's 64
    const float c0f = lif.charge_mode == CHARGE_IF ? 0.0f : 1.0f;
    const float c1f = lif.charge_mode == CHARGE_IF ? 1.0f : lif.inv_tau;
    const bool divide = lif.charge_mode == CHARGE_DIVIDE;   // tau is not a power of two: a true division

    float bias_row[NG];    // bias of this lane's channel row in each epilogue group; reloaded only when the wave moves to other channels
    int bias_ocf0 = -1;
    while (have_tile) {
        const int oc_tile = work - fast_div(work, g.d_oc_tiles) * g.oc_tiles;
        const int px_tile = px_tile_of(work);
        const int tile_y = fast_div(px_tile, g.d_tiles_x);
        const int tile_x = px_tile - tile_y * g.tiles_x;
        const int q0 = tile_y * g.TH;
        const int c0 = tile_x * g.TW;
        const int n_first = fast_div(q0, g.d_Ho);
        const int g_lo = n_first * g.H + (q0 - n_first * g.Ho) * g.sh - g.ph;
        int iw_lo = c0 * g.sw - g.pw;
        if (pair_shift && (iw_lo & 1)) iw_lo -= 1;

        // ---- matrix-operand view: this lane's two output pixels (2j, 2j + 1 of the wave's 64).
        bool pix_valid[kNPF];
        int ih0[kNPF], iw0[kNPF], lrow0[kNPF], lcol0[kNPF];
#pragma unroll
        for (int p = 0; p < kNPF; ++p) {
            const int pix = wm * (32 * kNPF) + (lane & 31) * kNPF + p;
            const int pr = fast_div(pix, g.d_TW);
            const int pc = pix - pr * g.TW;
            const int q = q0 + pr;
            const int ow = c0 + pc;
            pix_valid[p] = pr < g.TH && q < total_rows && ow < g.Wo;
            const int n = pix_valid[p] ? fast_div(q, g.d_Ho) : 0;
            const int oh = pix_valid[p] ? q - n * g.Ho : 0;
            ih0[p] = oh * g.sh - g.ph;
            iw0[p] = ow * g.sw - g.pw;
            lrow0[p] = n * g.H + ih0[p] - g_lo;
            lcol0[p] = iw0[p] - iw_lo;
        }

        // ---- epilogue view: 8 consecutive pixels of one channel row per lane; offsets walked incrementally.
        int pxoff[8];
        uint32_t okmask = 0;
        {
            const int pix0 = wm * (32 * kNPF) + pcx * 8;
            int pr = fast_div(pix0, g.d_TW);
            int pc = pix0 - pr * g.TW;
            int q = q0 + pr;
            int n = fast_div(q, g.d_Ho);
            int oh = q - n * g.Ho;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int ow = c0 + pc;
                const bool ok = pr < g.TH && q < total_rows && ow < g.Wo;
                pxoff[k] = ok ? (n * g.Cout * po + oh * g.Wo + ow) : 0;
                okmask |= ok ? (1u << k) : 0u;
                if (++pc == g.TW) {
                    pc = 0; ++pr; ++q;
                    if (++oh == g.Ho) { oh = 0; ++n; }
                }
            }
        }
        const bool fast = g.vec8 && okmask == 0xffu && (pxoff[7] - pxoff[0]) == 7 && (pxoff[0] & 7) == 0;

        const int ocf0 = (oc_tile << g.wn_log2) * NOF + wn * NOF;
        const bool wave_has_work = ocf0 < nocf;
        const uint16_t* __restrict__ wlane = wpacked + lane * 8;
        int64_t w_off[NOF];
#pragma unroll
        for (int f = 0; f < NOF; ++f) w_off[f] = static_cast<int64_t>(min(ocf0 + f, nocf - 1)) * frag_stride_ocf;
        if (g.w_lds && oc_tile != loaded_oc_tile) {
            // (Re)load the weight fragments of this output-channel tile into LDS; a workgroup normally keeps its tile.
            __syncthreads();
            const int frags_per_col = NOF * total_pairs;                 // 1 KiB fragments per wave column
            const int vec_total = (frags_per_col << g.wn_log2) * 64;     // 16-byte vectors
            for (int i = tid; i < vec_total; i += kConvThreads) {
                const int col = i / (frags_per_col * 64);
                const int rem = i - col * (frags_per_col * 64);
                const int f = rem / (total_pairs * 64);
                const int within = rem - f * (total_pairs * 64);          // pair * 64 + lane
                const int ocf = min(((oc_tile << g.wn_log2) + col) * NOF + f, nocf - 1);
                const cv_u32x4 val = *reinterpret_cast<const cv_u32x4*>(wpacked + static_cast<int64_t>(ocf) * frag_stride_ocf + static_cast<int64_t>(within) * 8);
                *reinterpret_cast<cv_u32x4*>(lds + tile_bytes + g.pitch + kToutStageBytes + static_cast<size_t>(i) * 16) = val;
            }
            loaded_oc_tile = oc_tile;
            __syncthreads();
        }
        const unsigned char* __restrict__ wl = wlds + (static_cast<size_t>(wn) * NOF * total_pairs * 64 + lane) * 16;

        // ---- membrane of this lane's 8 x 8 neurons (row group gi = f * 4 + kq), resident for all T steps.
        float v[NG][8];
        if (ocf0 != bias_ocf0) {
            bias_ocf0 = ocf0;
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int oc = (ocf0 + (gi >> 2)) * 32 + (gi & 3) * 8 + rg;
                bias_row[gi] = (wave_has_work && oc < g.Cout) ? bias[oc] : 0.0f;
            }
        }
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            const int oc = (ocf0 + (gi >> 2)) * 32 + (gi & 3) * 8 + rg;
            const bool row_ok = wave_has_work && oc < g.Cout && okmask != 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[gi][k] = 0.0f;
            if (row_ok && v_init != nullptr) {
                const int64_t row_off = static_cast<int64_t>(oc) * po;
                if (fast && g.v_is_f32) {
                    const float* src = static_cast<const float*>(v_init) + row_off + pxoff[0];
                    const Pack<float, 4> lo = *reinterpret_cast<const Pack<float, 4>*>(src);
                    const Pack<float, 4> hi = *reinterpret_cast<const Pack<float, 4>*>(src + 4);
#pragma unroll
                    for (int k = 0; k < 4; ++k) { v[gi][k] = lo.v[k]; v[gi][4 + k] = hi.v[k]; }
                } else {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        if (okmask & (1u << k)) {
                            v[gi][k] = g.v_is_f32 ? static_cast<const float*>(v_init)[row_off + pxoff[k]]
                                                  : to_float(static_cast<const XT*>(v_init)[row_off + pxoff[k]]);
                        }
                    }
                }
            }
        }

        cv_f32x16 acc[NOF][kNPF];
        cv_u32x4 a_cur[NOF], a_nxt[NOF];
#pragma unroll
        for (int f = 0; f < NOF; ++f) a_cur[f] = *reinterpret_cast<const cv_u32x4*>(wlane + w_off[f]);

        int next_work = work;
        bool next_tile = false;
        for (int step = 0; step < g.T; ++step) {
            if (step < steps_with_input) {
#pragma unroll
                for (int f = 0; f < NOF; ++f)
#pragma unroll
                    for (int p = 0; p < kNPF; ++p)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[f][p][r] = 0.0f;
                int gp = 0;
                for (int chunk = 0; chunk < g.nchunks; ++chunk) {
                    __syncthreads();   // every wave is done reading the previous stage from LDS
                    write_lds();       // waits for the prefetched loads
                    __syncthreads();
                    // ---- put the next stage's loads in flight: next chunk, next timestep, or the next tile.
                    if (chunk + 1 < g.nchunks) {
                        issue_loads(step, chunk + 1);
                    } else if (step + 1 < steps_with_input) {
                        issue_loads(step + 1, 0);
                    } else {
                        next_work = work + slots_per_xcd;
                        next_tile = next_work < work_per_xcd && px_tile_of(next_work) < n_px_tiles;
                        if (next_tile) {
                            compute_descriptors(px_tile_of(next_work));
                            issue_loads(0, 0);
                        }
                    }
                    if (!wave_has_work) continue;
                    int cg = half & (groups - 1);
                    int kh = 0, kw = 0;
                    if (half >> g.groups_log2) { kw = 1; if (kw == g.KW) { kw = 0; kh = 1; } }
                    int tap_off[kNPF];   // LDS offset of this lane's pixel for the current tap, -1 = outside the input
#pragma unroll
                    for (int p = 0; p < kNPF; ++p) {
                        const bool ok = pix_valid[p] && kh < g.KH && static_cast<unsigned>(ih0[p] + kh) < static_cast<unsigned>(g.H) &&
                                        static_cast<unsigned>(iw0[p] + kw) < static_cast<unsigned>(g.W);
                        tap_off[p] = ok ? ((lrow0[p] + kh) * g.WT + lcol0[p] + kw) * g.pitch : -1;
                    }
                    if (g.w_lds) {
                        for (int pair = 0; pair < g.npairs; ++pair, ++gp) {
    #pragma unroll
                            for (int f = 0; f < NOF; ++f)
                                a_cur[f] = *reinterpret_cast<const cv_u32x4*>(wl + (static_cast<size_t>(f) * total_pairs + gp) * kFragBytes);
                            cv_u32x4 b[kNPF];
    #pragma unroll
                            for (int p = 0; p < kNPF; ++p)
                                b[p] = *reinterpret_cast<const cv_u32x4*>(lds + (tap_off[p] >= 0 ? tap_off[p] + cg * 16 : zero_off));
    #pragma unroll
                            for (int f = 0; f < NOF; ++f)
    #pragma unroll
                                for (int p = 0; p < kNPF; ++p) acc[f][p] = cv_mfma<F16>(a_cur[f], b[p], acc[f][p]);
                            cg += 2;
                            if (cg >= groups) {
                                do {
                                    cg -= groups;
                                    if (++kw == g.KW) { kw = 0; ++kh; }
                                } while (cg >= groups);
    #pragma unroll
                                for (int p = 0; p < kNPF; ++p) {
                                    const bool ok = pix_valid[p] && kh < g.KH && static_cast<unsigned>(ih0[p] + kh) < static_cast<unsigned>(g.H) &&
                                                    static_cast<unsigned>(iw0[p] + kw) < static_cast<unsigned>(g.W);
                                    tap_off[p] = ok ? ((lrow0[p] + kh) * g.WT + lcol0[p] + kw) * g.pitch : -1;
                                }
                            }
                        }
                    } else {
                        for (int pair = 0; pair < g.npairs; ++pair, ++gp) {
                            const int gp_next = gp + 1 < total_pairs ? gp + 1 : 0;   // wraps to the next timestep's first pair
    #pragma unroll
                            for (int f = 0; f < NOF; ++f)
                                a_nxt[f] = *reinterpret_cast<const cv_u32x4*>(wlane + w_off[f] + static_cast<int64_t>(gp_next) * (kFragBytes / 2));
                            cv_u32x4 b[kNPF];
    #pragma unroll
                            for (int p = 0; p < kNPF; ++p)
                                b[p] = *reinterpret_cast<const cv_u32x4*>(lds + (tap_off[p] >= 0 ? tap_off[p] + cg * 16 : zero_off));
    #pragma unroll
                            for (int f = 0; f < NOF; ++f)
    #pragma unroll
                                for (int p = 0; p < kNPF; ++p) acc[f][p] = cv_mfma<F16>(a_cur[f], b[p], acc[f][p]);
    #pragma unroll
                            for (int f = 0; f < NOF; ++f) a_cur[f] = a_nxt[f];
                            cg += 2;
                            if (cg >= groups) {
                                do {
                                    cg -= groups;
                                    if (++kw == g.KW) { kw = 0; ++kh; }
                                } while (cg >= groups);
    #pragma unroll
                                for (int p = 0; p < kNPF; ++p) {
                                    const bool ok = pix_valid[p] && kh < g.KH && static_cast<unsigned>(ih0[p] + kh) < static_cast<unsigned>(g.H) &&
                                                    static_cast<unsigned>(iw0[p] + kw) < static_cast<unsigned>(g.W);
                                    tap_off[p] = ok ? ((lrow0[p] + kh) * g.WT + lcol0[p] + kw) * g.pitch : -1;
                                }
                            }
                        }
                    }
                }
            }

            // ---- LIF step on this wave's 64 x 64 outputs: transpose 8 channel rows at a time through the wave's stage.
            if (wave_has_work) {
                XT* __restrict__ out_t = spikes + step * g.spike_step_stride;
                const XT* __restrict__ res_t = has_residual ? static_cast<const XT*>(step_pointer(residuals, step)) : nullptr;
#pragma unroll
                for (int gi = 0; gi < NG; ++gi) {
                    const int f = gi >> 2, kq = gi & 3;
                    __builtin_amdgcn_wave_barrier();
                    // stage layout [pixel][8 channel rows]: a lane's 4 consecutive accumulator rows go out as one 16-byte write.
#pragma unroll
                    for (int p = 0; p < kNPF; ++p) {
                        const Pack<float, 4> four = {{acc[f][p][kq * 4 + 0], acc[f][p][kq * 4 + 1], acc[f][p][kq * 4 + 2], acc[f][p][kq * 4 + 3]}};
                        *reinterpret_cast<Pack<float, 4>*>(stage + ((lane & 31) * kNPF + p) * kToutStagePitch + half * 4) = four;
                    }
                    __builtin_amdgcn_wave_barrier();
                    const int oc = (ocf0 + f) * 32 + kq * 8 + rg;
                    if (oc < g.Cout && okmask != 0) {
                        float x[8];
#pragma unroll
                        for (int k = 0; k < 8; ++k) x[k] = stage[(pcx * 8 + k) * kToutStagePitch + rg] + bias_row[gi];
                        const int64_t row_off = static_cast<int64_t>(oc) * po;
                        if (res_t != nullptr) {
                            if (fast) {
                                const Pack<XT, 8> rr8 = *reinterpret_cast<const Pack<XT, 8>*>(res_t + row_off + pxoff[0]);
#pragma unroll
                                for (int k = 0; k < 8; ++k) x[k] += to_float(rr8.v[k]);
                            } else {
#pragma unroll
                                for (int k = 0; k < 8; ++k)
                                    if (okmask & (1u << k)) x[k] += to_float(res_t[row_off + pxoff[k]]);
                            }
                        }
                        Pack<XT, 8> sp;
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            bool fired;
                            if constexpr (STD) {
                                const float h = v[gi][k] + (x[k] - v[gi][k]) * lif.inv_tau;
                                fired = h >= lif.v_threshold;
                                v[gi][k] = fired ? lif.v_reset : h;
                            } else {
                                const float h = divide ? v[gi][k] + __fdiv_rn(x[k] - v[gi][k], lif.tau) : v[gi][k] + (x[k] - v[gi][k] * c0f) * c1f;
                                fired = h >= lif.v_threshold;
                                v[gi][k] = fired ? (lif.soft_reset ? h - lif.v_threshold : lif.v_reset) : h;
                            }
                            sp.v[k] = spike_value<XT>(fired);
                        }
                        if (fast) {
                            *reinterpret_cast<Pack<XT, 8>*>(out_t + row_off + pxoff[0]) = sp;
                        } else {
#pragma unroll
                            for (int k = 0; k < 8; ++k)
                                if (okmask & (1u << k)) out_t[row_off + pxoff[k]] = sp.v[k];
                        }
                    }
                }
            }
        }

        // ---- final membrane.
        if (wave_has_work && okmask != 0) {
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int oc = (ocf0 + (gi >> 2)) * 32 + (gi & 3) * 8 + rg;
                if (oc < g.Cout) {
                    const int64_t row_off = static_cast<int64_t>(oc) * po;
                    if (fast && g.v_is_f32) {
                        float* dst = static_cast<float*>(v_out) + row_off + pxoff[0];
                        Pack<float, 4> lo, hi;
#pragma unroll
                        for (int k = 0; k < 4; ++k) { lo.v[k] = v[gi][k]; hi.v[k] = v[gi][4 + k]; }
                        *reinterpret_cast<Pack<float, 4>*>(dst) = lo;
                        *reinterpret_cast<Pack<float, 4>*>(dst + 4) = hi;
                    } else {
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            if (okmask & (1u << k)) {
                                if (g.v_is_f32) static_cast<float*>(v_out)[row_off + pxoff[k]] = v[gi][k];
                                else static_cast<XT*>(v_out)[row_off + pxoff[k]] = from_float<XT>(v[gi][k]);
                            }
                        }
                    }
                }
            }
        }
        work = next_work;
        have_tile = next_tile;
    }
}

template <typename XT>
int launch_conv_tout(const ConvLaunch& L, int load_mode) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kConvThreads, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.has_residual, L.g, L.wpacked, L.bias, L.v_init,
                                                                      static_cast<XT*>(L.spikes), L.v_out, L.lif);
        return check_launch("snnf_conv_lif");
    };
    const bool std_lif = L.lif.charge_mode == CHARGE_SCALE && !L.lif.soft_reset;
    if constexpr (sizeof(XT) == 4) {
        return std_lif ? run(conv_lif_tout_kernel<XT, LOAD_2XF32, true>) : run(conv_lif_tout_kernel<XT, LOAD_2XF32, false>);
    } else {
        if (load_mode == LOAD_PAIR32)
            return std_lif ? run(conv_lif_tout_kernel<XT, LOAD_PAIR32, true>) : run(conv_lif_tout_kernel<XT, LOAD_PAIR32, false>);
        return std_lif ? run(conv_lif_tout_kernel<XT, LOAD_2X16, true>) : run(conv_lif_tout_kernel<XT, LOAD_2X16, false>);
    }
}

}  // namespace snnf
