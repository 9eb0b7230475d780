// Dense convolution + bias (+ residual) + LIF over T timesteps as an implicit GEMM on the gfx950 matrix cores.
//
//   out^T[Cout, T * pixels] = Wp[Cout, K] . im2col(x)[K, T * pixels],   K = taps * Cin,   then LIF along T per neuron.
//
// Mapping (v_mfma_f32_32x32x16, fp32 accumulate):
//   * M = output channels (A operand = weights), N = output pixels (B operand = activations). A wave owns 64 channels
//     x 64 pixels x TT timesteps of accumulators; a lane of the result owns two ADJACENT pixels of 16 channels per
//     fragment, so spikes leave as 4-byte stores and membranes as 8-byte stores.
//   * All TT timesteps of a pixel tile are accumulated side by side: one weight fragment load feeds TT * 2 matrix
//     operations and the LIF recurrence runs in the epilogue on accumulators that never leave registers.
//   * Weights are pre-packed in fragment order: a 32x16 weight fragment is one contiguous 1 KiB global load straight
//     into registers (prefetched one step ahead); a layer's packed weights stay L2 resident.
//   * Activations (NCHW, pixel-contiguous) are transposed on the way into LDS to [pixel][channel], 8 channels per
//     16-byte group = the per-lane operand order of the matrix instruction. A halo tile is staged once per channel
//     chunk and re-read for every tap with a per-lane pixel offset; padding and image borders redirect the lane to a
//     zero pixel.
//   * Workgroups are persistent: each walks a list of tiles and issues the global loads of the next stage (next channel
//     chunk, or the first chunk of its next tile) before the matrix work and the epilogue of the current one, so HBM
//     reads overlap compute and stores. Staging addresses are computed once per tile, not per chunk.
//   * Tile order keeps the workgroups that share a pixel tile (different output-channel tiles) on one XCD.
#pragma once

#include "snnf_conv_common.h"

namespace snnf {

typedef __bf16 cv_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 cv_f16x8 __attribute__((ext_vector_type(8)));
typedef float cv_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t cv_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t cv_u32x2 __attribute__((ext_vector_type(2)));
typedef float cv_f32x2 __attribute__((ext_vector_type(2)));

template <bool F16>
__device__ __forceinline__ cv_f32x16 cv_mfma(cv_u32x4 a, cv_u32x4 b, cv_f32x16 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(cv_f16x8, a), __builtin_bit_cast(cv_f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(cv_bf16x8, a), __builtin_bit_cast(cv_bf16x8, b), c, 0, 0, 0);
    }
}

template <typename XT, int TT, int LM>
__global__ __launch_bounds__(kConvThreads) void conv_lif_kernel(const StepPtrs xs, const StepPtrs residuals,
                                                                const int has_residual, const ConvGeom g,
                                                                const uint16_t* __restrict__ wpacked,
                                                                const float* __restrict__ bias,
                                                                const void* __restrict__ v_init,
                                                                XT* __restrict__ spikes, void* __restrict__ v_out,
                                                                const LifParams lif) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    constexpr int RPE = LM == LOAD_PAIR32 ? 1 : 2;     // prefetch registers per (channel, pixel pair)
    constexpr int MI = staging_items(LM);              // staging items per thread and chunk
    constexpr int SS = MI / TT;                        // spatial staging slots per thread
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int wm = wave & ((1 << g.wm_log2) - 1);
    const int wn = wave >> g.wm_log2;

    const int groups = 1 << g.groups_log2;
    const int tile_bytes = g.NR * g.WT * g.pitch;
    const int t_in = g.shared_x ? 1 : TT;
    const int zero_off = max(t_in * tile_bytes, static_cast<int>(kEpiBytes));   // the epilogue stage shares the tile's LDS
    const int total_rows = g.N * g.Ho;
    const int64_t plane = static_cast<int64_t>(g.H) * g.W;
    const int64_t plane_out = static_cast<int64_t>(g.Ho) * g.Wo;
    const int WTP = g.WT >> 1;
    const bool pair_shift = LM == LOAD_PAIR32;  // tile columns start at an even input column
    const int nocf = (g.Cout + 31) >> 5;
    const int64_t frag_stride_ocf = static_cast<int64_t>(g.nchunks) * g.npairs * (kFragBytes / 2);
    const int total_pairs = g.nchunks * g.npairs;

    if (tid < g.pitch / 4) reinterpret_cast<uint32_t*>(lds + zero_off)[tid] = 0u;

    // ---- persistent tile walk: XCD x handles pixel tiles = x (mod 8); consecutive slots take the oc tiles of one pixel tile.
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int slots_per_xcd = gridDim.x >> 3;
    const int n_px_tiles = g.tiles_x * g.tiles_y;
    const int px_per_xcd = (n_px_tiles + 7) >> 3;
    const int work_per_xcd = px_per_xcd * g.oc_tiles;

    // ---- staging descriptors of the NEXT stage to load (recomputed per tile). A slot covers 8 channels x 2 adjacent
    // input columns for every timestep; its source is addressed as (uniform base pointer) + (32-bit per-lane offset).
    uint32_t st_src[SS];   // byte offset of (chunk 0, channel group, row, SECOND column of the pair) in a timestep tensor
    uint32_t st_meta[SS];  // LDS byte offset in a timestep tile | flags << 20 | channel group << 24
                           // flags: bit0 first column valid, bit1 second column valid, bit2 slot exists and row is inside
    uint32_t pre[MI][8][RPE];
    constexpr int ES = static_cast<int>(sizeof(XT));

    auto compute_descriptors = [&](int px_tile) __attribute__((always_inline)) {
        const int tile_x = px_tile % g.tiles_x;
        const int tile_y = px_tile / g.tiles_x;
        const int q0 = tile_y * g.TH;
        const int q_last = min(q0 + g.TH, total_rows) - 1;
        const int n_first = q0 / g.Ho;
        const int g_lo = n_first * g.H + (q0 - n_first * g.Ho) * g.sh - g.ph;
        const int n_last = q_last / g.Ho;
        const int rows = n_last * g.H + (q_last - n_last * g.Ho) * g.sh - g.ph + g.KH - g_lo;
        int iw_lo = tile_x * g.TW * g.sw - g.pw;
        if (pair_shift && (iw_lo & 1)) iw_lo -= 1;
        const int spatial_items = groups * rows * WTP;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            const int e = s * kConvThreads + tid;
            int flags = 0, src = 0, dst = 0, cg = 0;
            if (e < spatial_items) {
                cg = e / (rows * WTP);
                const int rem = e - cg * (rows * WTP);
                const int r = rem / WTP;
                const int cp = rem - r * WTP;
                const int grow = g_lo + r;
                const int iw = iw_lo + cp * 2;
                dst = (r * g.WT + cp * 2) * g.pitch + cg * 16;
                if (grow >= 0 && grow < g.N * g.H) {
                    const int xn = grow / g.H;
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
    auto issue_loads = [&](int chunk) __attribute__((always_inline)) {
        if constexpr (LM == LOAD_2XF32) split_chunk(chunk, g.nchunks_r, pre_part, chunk);
        const int64_t chunk_bytes = static_cast<int64_t>(chunk) * g.CK * plane * ES;
#pragma unroll
        for (int u = 0; u < MI; ++u) {
            const int t = u % TT;
            const int s = u / TT;
            const uint32_t flags = st_meta[s] >> 20;
            if (t < t_in && (flags & 4)) {
                const char* __restrict__ base = static_cast<const char*>(xs.p[t]) + chunk_bytes;  // uniform
                const int nval = g.Cin - (chunk * g.CK + static_cast<int>((st_meta[s] >> 24) & 31u) * 8);
                const bool ok0 = flags & 1, ok1 = flags & 2;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const bool cok = j < nval;
                    const char* __restrict__ row = base + j * plane * ES;  // uniform
                    if constexpr (LM == LOAD_PAIR32) {
                        pre[u][j][0] = (cok && ok0) ? *reinterpret_cast<const uint32_t*>(row + st_src[s] - 2) : 0u;
                    } else if constexpr (LM == LOAD_2X16) {
                        pre[u][j][0] = (cok && ok0) ? *reinterpret_cast<const uint16_t*>(row + st_src[s] - 2) : 0u;
                        pre[u][j][1] = (cok && ok1) ? *reinterpret_cast<const uint16_t*>(row + st_src[s]) : 0u;
                    } else {
                        pre[u][j][0] = (cok && ok0) ? *reinterpret_cast<const uint32_t*>(row + st_src[s] - 4) : 0u;
                        pre[u][j][1] = (cok && ok1) ? *reinterpret_cast<const uint32_t*>(row + st_src[s]) : 0u;
                    }
                }
            }
        }
    };

    auto write_lds = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < MI; ++u) {
            const int t = u % TT;
            const int s = u / TT;
            if (t < t_in && ((st_meta[s] >> 20) & 4)) {
                uint32_t e0[8], e1[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if constexpr (LM == LOAD_PAIR32) {
                        e0[j] = pre[u][j][0] & 0xffffu;
                        e1[j] = pre[u][j][0] >> 16;
                    } else if constexpr (LM == LOAD_2X16) {
                        e0[j] = pre[u][j][0];
                        e1[j] = pre[u][j][1];
                    } else {
                        e0[j] = split_bf16_bits(__uint_as_float(pre[u][j][0]), pre_part == 2);
                        e1[j] = split_bf16_bits(__uint_as_float(pre[u][j][1]), pre_part == 2);
                    }
                }
                cv_u32x4 lo, hi;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    lo[k] = e0[2 * k] | (e0[2 * k + 1] << 16);
                    hi[k] = e1[2 * k] | (e1[2 * k + 1] << 16);
                }
                unsigned char* dst = lds + t * tile_bytes + (st_meta[s] & 0xfffffu);
                *reinterpret_cast<cv_u32x4*>(dst) = lo;
                *reinterpret_cast<cv_u32x4*>(dst + g.pitch) = hi;
            }
        }
    };

    int work = slot;                     // index into this XCD's work list
    auto px_tile_of = [&](int w) __attribute__((always_inline)) { return (w / g.oc_tiles) * 8 + xcd; };
    bool have_tile = work < work_per_xcd && px_tile_of(work) < n_px_tiles;
    if (have_tile) {
        compute_descriptors(px_tile_of(work));
        issue_loads(0);
    }

    while (have_tile) {
        const int oc_tile = work % g.oc_tiles;
        const int px_tile = px_tile_of(work);
        const int tile_x = px_tile % g.tiles_x;
        const int tile_y = px_tile / g.tiles_x;
        const int q0 = tile_y * g.TH;
        const int c0 = tile_x * g.TW;
        const int n_first = q0 / g.Ho;
        const int g_lo = n_first * g.H + (q0 - n_first * g.Ho) * g.sh - g.ph;
        int iw_lo = c0 * g.sw - g.pw;
        if (pair_shift && (iw_lo & 1)) iw_lo -= 1;

        // ---- this lane's two output pixels.
        bool pix_valid[kNPF];
        int ih0[kNPF], iw0[kNPF], lrow0[kNPF], lcol0[kNPF];
        int64_t pix_off[kNPF];
#pragma unroll
        for (int p = 0; p < kNPF; ++p) {
            const int pix = wm * (32 * kNPF) + (lane & 31) * kNPF + p;
            const int pr = pix / g.TW;
            const int pc = pix - pr * g.TW;
            const int q = q0 + pr;
            const int ow = c0 + pc;
            pix_valid[p] = pr < g.TH && q < total_rows && ow < g.Wo;
            const int n = pix_valid[p] ? q / g.Ho : 0;
            const int oh = pix_valid[p] ? q - n * g.Ho : 0;
            ih0[p] = oh * g.sh - g.ph;
            iw0[p] = ow * g.sw - g.pw;
            lrow0[p] = n * g.H + ih0[p] - g_lo;
            lcol0[p] = iw0[p] - iw_lo;
            pix_off[p] = static_cast<int64_t>(n) * g.Cout * plane_out + static_cast<int64_t>(oh) * g.Wo + ow;
        }

        cv_f32x16 acc[TT][kNOF][kNPF];
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int f = 0; f < kNOF; ++f)
#pragma unroll
                for (int p = 0; p < kNPF; ++p)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[t][f][p][r] = 0.0f;

        const int ocf0 = (oc_tile << g.wn_log2) * kNOF + wn * kNOF;
        const bool wave_has_work = ocf0 < nocf;
        const uint16_t* __restrict__ wlane = wpacked + lane * 8;
        int64_t w_off[kNOF];
#pragma unroll
        for (int f = 0; f < kNOF; ++f) w_off[f] = static_cast<int64_t>(min(ocf0 + f, nocf - 1)) * frag_stride_ocf;

        cv_u32x4 a_cur[kNOF], a_nxt[kNOF];
#pragma unroll
        for (int f = 0; f < kNOF; ++f) a_cur[f] = *reinterpret_cast<const cv_u32x4*>(wlane + w_off[f]);

        int next_work = work;
        bool next_tile = false;
        int gp = 0;  // global pair index = chunk * npairs + pair
        for (int chunk = 0; chunk < g.nchunks; ++chunk) {
            __syncthreads();   // every wave is done reading the previous stage from LDS
            write_lds();       // waits for the prefetched loads
            __syncthreads();
            // ---- put the next stage's loads in flight.
            if (chunk + 1 < g.nchunks) {
                issue_loads(chunk + 1);
            } else {
                next_work = work + slots_per_xcd;
                next_tile = next_work < work_per_xcd && px_tile_of(next_work) < n_px_tiles;
                if (next_tile) {
                    compute_descriptors(px_tile_of(next_work));
                    issue_loads(0);
                }
            }
            if (!wave_has_work) {
                gp += g.npairs;
                continue;
            }
            // ---- matrix work of this chunk: slot s = 2 * pair + half -> (tap, channel group).
            int cg = half & (groups - 1);
            int kh = 0, kw = 0;
            if (half >> g.groups_log2) { kw = 1; if (kw == g.KW) { kw = 0; kh = 1; } }
            for (int pair = 0; pair < g.npairs; ++pair, ++gp) {
                if (gp + 1 < total_pairs) {
#pragma unroll
                    for (int f = 0; f < kNOF; ++f)
                        a_nxt[f] = *reinterpret_cast<const cv_u32x4*>(wlane + w_off[f] + static_cast<int64_t>(gp + 1) * (kFragBytes / 2));
                }
                int off[kNPF];
#pragma unroll
                for (int p = 0; p < kNPF; ++p) {
                    const bool ok = pix_valid[p] && kh < g.KH && static_cast<unsigned>(ih0[p] + kh) < static_cast<unsigned>(g.H) &&
                                    static_cast<unsigned>(iw0[p] + kw) < static_cast<unsigned>(g.W);
                    off[p] = ok ? ((lrow0[p] + kh) * g.WT + lcol0[p] + kw) * g.pitch + cg * 16 : -1;
                }
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    if (t < t_in) {
                        cv_u32x4 b[kNPF];
#pragma unroll
                        for (int p = 0; p < kNPF; ++p)
                            b[p] = *reinterpret_cast<const cv_u32x4*>(lds + (off[p] >= 0 ? t * tile_bytes + off[p] : zero_off));
#pragma unroll
                        for (int f = 0; f < kNOF; ++f)
#pragma unroll
                            for (int p = 0; p < kNPF; ++p) acc[t][f][p] = cv_mfma<F16>(a_cur[f], b[p], acc[t][f][p]);
                    }
                }
#pragma unroll
                for (int f = 0; f < kNOF; ++f) a_cur[f] = a_nxt[f];
                cg += 2;
                while (cg >= groups) {
                    cg -= groups;
                    if (++kw == g.KW) { kw = 0; ++kh; }
                }
            }
        }

        // ---- epilogue. Eight channel rows at a time, the accumulators of all T steps are transposed through LDS (the
        // activation tile is dead by now) to [step][channel row][64 pixels] per wave, so that a lane owns 8 consecutive
        // pixels of one channel: bias (+ residual) + LIF run on those 8 neurons with the membrane in registers across
        // the T steps, spikes leave as one 16-byte store per step and the membrane as two. Branch-free neuron:
        // h = v + (x - v * c0) * c1 covers tau <= 1 (c0 = 0, c1 = 1) and power-of-two tau exactly.
        __syncthreads();   // every wave is done reading the activation tile
        if (g.shared_x) {
#pragma unroll
            for (int t = 1; t < TT; ++t)
#pragma unroll
                for (int f = 0; f < kNOF; ++f)
#pragma unroll
                    for (int p = 0; p < kNPF; ++p) acc[t][f][p] = acc[0][f][p];
        }
        if (wave_has_work) {
            float* __restrict__ stage = reinterpret_cast<float*>(lds) + wave * (TT * 8 * kEpiPitch);
            const int rg = lane >> 3;            // channel row of this lane inside a group of 8
            const int pcx = lane & 7;            // pixel chunk: pixels 8 * pcx .. 8 * pcx + 7 of the wave's 64
            // Output offsets (elements, inside one channel plane stack) of the chunk's pixels, walked incrementally.
            int pxoff[8];
            uint32_t okmask = 0;
            {
                const int pix0 = wm * (32 * kNPF) + pcx * 8;
                int pr = pix0 / g.TW;
                int pc = pix0 - pr * g.TW;
                int q = q0 + pr;
                int n = q / g.Ho;
                int oh = q - n * g.Ho;
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int ow = c0 + pc;
                    const bool ok = pr < g.TH && q < total_rows && ow < g.Wo;
                    pxoff[k] = ok ? (n * g.Cout * static_cast<int>(plane_out) + oh * g.Wo + ow) : 0;
                    okmask |= ok ? (1u << k) : 0u;
                    if (++pc == g.TW) {
                        pc = 0; ++pr; ++q;
                        if (++oh == g.Ho) { oh = 0; ++n; }
                    }
                }
            }
            const bool fast = g.vec8 && okmask == 0xffu && (pxoff[7] - pxoff[0]) == 7 && (pxoff[0] & 7) == 0;
            const float c0f = lif.charge_mode == CHARGE_IF ? 0.0f : 1.0f;
            const float c1f = lif.charge_mode == CHARGE_IF ? 1.0f : lif.inv_tau;
            const bool divide = lif.charge_mode == CHARGE_DIVIDE;   // tau is not a power of two: a true division
            const int po = static_cast<int>(plane_out);

#pragma unroll
            for (int f = 0; f < kNOF; ++f) {
#pragma unroll
                for (int kq = 0; kq < 4; ++kq) {
                    // rows of this group: channel (ocf0 + f) * 32 + 8 * kq + [0, 8); lane (j, half) holds rows 4 * half + (r & 3).
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int t = 0; t < TT; ++t)
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) {
                            const cv_f32x2 two = {acc[t][f][0][kq * 4 + rr], acc[t][f][1][kq * 4 + rr]};
                            *reinterpret_cast<cv_f32x2*>(stage + (t * 8 + half * 4 + rr) * kEpiPitch + (lane & 31) * 2) = two;
                        }
                    __builtin_amdgcn_wave_barrier();
                    const int oc = (ocf0 + f) * 32 + kq * 8 + rg;
                    if (oc < g.Cout && okmask != 0) {
                        const int64_t row_off = static_cast<int64_t>(oc) * po;
                        const float bvv = bias[oc];
                        float v[8];
#pragma unroll
                        for (int k = 0; k < 8; ++k) v[k] = 0.0f;
                        if (v_init != nullptr) {
                            if (fast && g.v_is_f32) {
                                const float* src = static_cast<const float*>(v_init) + row_off + pxoff[0];
                                const Pack<float, 4> lo = *reinterpret_cast<const Pack<float, 4>*>(src);
                                const Pack<float, 4> hi = *reinterpret_cast<const Pack<float, 4>*>(src + 4);
#pragma unroll
                                for (int k = 0; k < 4; ++k) { v[k] = lo.v[k]; v[4 + k] = hi.v[k]; }
                            } else {
#pragma unroll
                                for (int k = 0; k < 8; ++k) {
                                    if (okmask & (1u << k)) {
                                        v[k] = g.v_is_f32 ? static_cast<const float*>(v_init)[row_off + pxoff[k]]
                                                          : to_float(static_cast<const XT*>(v_init)[row_off + pxoff[k]]);
                                    }
                                }
                            }
                        }
#pragma unroll
                        for (int t = 0; t < TT; ++t) {
                            if (t < g.T) {
                                const float* __restrict__ srow = stage + (t * 8 + rg) * kEpiPitch + pcx * 8;
                                const Pack<float, 4> xlo = *reinterpret_cast<const Pack<float, 4>*>(srow);
                                const Pack<float, 4> xhi = *reinterpret_cast<const Pack<float, 4>*>(srow + 4);
                                float x[8];
#pragma unroll
                                for (int k = 0; k < 4; ++k) { x[k] = xlo.v[k] + bvv; x[4 + k] = xhi.v[k] + bvv; }
                                XT* __restrict__ out_t = spikes + t * g.spike_step_stride + row_off;
                                if (has_residual) {
                                    const XT* __restrict__ res_t = static_cast<const XT*>(residuals.p[t]) + row_off;
                                    if (fast) {
                                        const Pack<XT, 8> rr8 = *reinterpret_cast<const Pack<XT, 8>*>(res_t + pxoff[0]);
#pragma unroll
                                        for (int k = 0; k < 8; ++k) x[k] += to_float(rr8.v[k]);
                                    } else {
#pragma unroll
                                        for (int k = 0; k < 8; ++k)
                                            if (okmask & (1u << k)) x[k] += to_float(res_t[pxoff[k]]);
                                    }
                                }
                                Pack<XT, 8> sp;
#pragma unroll
                                for (int k = 0; k < 8; ++k) {
                                    const float h = divide ? v[k] + __fdiv_rn(x[k] - v[k], lif.tau) : v[k] + (x[k] - v[k] * c0f) * c1f;
                                    const bool fired = h >= lif.v_threshold;
                                    v[k] = fired ? (lif.soft_reset ? h - lif.v_threshold : lif.v_reset) : h;
                                    sp.v[k] = spike_value<XT>(fired);
                                }
                                if (fast) {
                                    *reinterpret_cast<Pack<XT, 8>*>(out_t + pxoff[0]) = sp;
                                } else {
#pragma unroll
                                    for (int k = 0; k < 8; ++k)
                                        if (okmask & (1u << k)) out_t[pxoff[k]] = sp.v[k];
                                }
                            }
                        }
                        if (fast && g.v_is_f32) {
                            float* dst = static_cast<float*>(v_out) + row_off + pxoff[0];
                            Pack<float, 4> lo, hi;
#pragma unroll
                            for (int k = 0; k < 4; ++k) { lo.v[k] = v[k]; hi.v[k] = v[4 + k]; }
                            *reinterpret_cast<Pack<float, 4>*>(dst) = lo;
                            *reinterpret_cast<Pack<float, 4>*>(dst + 4) = hi;
                        } else {
#pragma unroll
                            for (int k = 0; k < 8; ++k) {
                                if (okmask & (1u << k)) {
                                    if (g.v_is_f32) static_cast<float*>(v_out)[row_off + pxoff[k]] = v[k];
                                    else static_cast<XT*>(v_out)[row_off + pxoff[k]] = from_float<XT>(v[k]);
                                }
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

template <typename XT, int TT>
int launch_conv_lm(const ConvLaunch& L, int load_mode) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kConvThreads, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.has_residual, L.g, L.wpacked, L.bias, L.v_init,
                                                                      static_cast<XT*>(L.spikes), L.v_out, L.lif);
        return check_launch("snnf_conv_lif");
    };
    if constexpr (sizeof(XT) == 4) {
        return run(conv_lif_kernel<XT, TT, LOAD_2XF32>);
    } else {
        if (load_mode == LOAD_PAIR32) return run(conv_lif_kernel<XT, TT, LOAD_PAIR32>);
        return run(conv_lif_kernel<XT, TT, LOAD_2X16>);
    }
}

template <typename XT>
int launch_conv_tt(const ConvLaunch& L, int tt, int load_mode) {
    if (tt == 1) return launch_conv_lm<XT, 1>(L, load_mode);
    if (tt == 2) return launch_conv_lm<XT, 2>(L, load_mode);
    return launch_conv_lm<XT, 4>(L, load_mode);
}

}  // namespace snnf
