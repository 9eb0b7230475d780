// Pointwise (1x1, stride 1, no padding) convolution + bias (+ residual) + LIF over T timesteps.
//
// A pointwise layer moves far more bytes than it multiplies (its roofline is HBM), and on this machine a wave64
// vector instruction occupies its SIMD for four cycles, so what decides the speed of this kernel is the number of
// vector instructions per output and the waits on memory, not the matrix work. Hence:
//   * an image is one row of P = H * W pixels; a tile is 64 consecutive pixels x 128 output channels (4 waves x 32).
//     Per-thread staging offsets, LDS addresses of the matrix operands and output offsets are kernel constants; a tile
//     only contributes a uniform base address, so loads and stores use the scalar-base addressing form.
//   * The bias enters through the matrix unit (a fragment holding the fp32 bias split into three 16-bit terms times a
//     fragment of ones), so a timestep starts with one matrix instruction instead of clearing and biasing registers.
//   * The membrane of the wave's 32 x 64 neurons stays in registers for all T. Timestep pointers are read from the
//     kernel-argument segment with a scalar load instead of living in 32 scalar registers per table.
//   * One counter tracks all of a wave's outstanding global loads and stores, in order. The next stage's loads are
//     issued from a single place in the loop (copies between two sets of load registers would force a wait right after
//     the loads), and a timestep's spikes wait in registers until the next stage has been taken out of its load
//     registers, so that the wait for those loads never finds fresh stores in front of it.
//   * The activation tile is double buffered in LDS when it fits (one workgroup barrier per stage). A wave's weight
//     fragments stay in registers when there are exactly 8 of them (Cin of 113..128), else the workgroup's fragments stay in
//     LDS when they fit, else they stream from L2 one fragment ahead. LDS bandwidth is the next limit after the vector
//     unit, so LDS rows are laid out for conflict-free 16-byte reads.
// FAST: every tile of the launch lies inside its image, outputs are 16-byte aligned, Cout % 32 == 0 and the membrane is
// fp32, so the per-pixel and per-row masks and the element-wise load/store paths (and the scalar registers they pin)
// drop out; the host sends the ragged last tile of each image, and any layer that fails these conditions, to the
// general variant. Requires Cin % 8 == 0 (channel groups of 8 are whole). Operand mapping and the packed weight format are those of
// snnf_conv_kernel.h.
#pragma once

#include <type_traits>

#include "snnf_conv_kernel.h"

namespace snnf {

constexpr int kPwStagePitch = 68;                          // floats per channel row of the wave's stage (64 pixels + padding)
constexpr int kPwStageFloats = 8 * kPwStagePitch;          // 8 channel rows
static_assert(4 * kPwStageFloats * sizeof(float) == kPwStageBytes, "host and kernel disagree on the stage size");
constexpr int kPwTile = 64;                                // pixels per tile
constexpr int kPwSlots = 2;                                // staging items per thread and chunk (128 channels x 64 pixels)
constexpr int kPwRegPairs = 8;                             // weight fragments a wave can keep in registers

enum PwWeights : int { PW_WEIGHTS_STREAM = 0, PW_WEIGHTS_LDS = 1, PW_WEIGHTS_REGS = 2 };

// Entry i of a pointer table passed by value as a kernel argument, read from the kernel-argument segment (explicit
// arguments start at offset 0 of that segment, in declaration order and naturally aligned).
typedef const void* pw_cvp;
__device__ __forceinline__ const void* kernarg_table_entry(int table_offset_bytes, int i) {
    typedef const __attribute__((address_space(4))) unsigned char* ka_bytes;
    typedef const __attribute__((address_space(4))) pw_cvp* ka_entry;
    ka_bytes ka = (ka_bytes)__builtin_amdgcn_kernarg_segment_ptr();
    return *(ka_entry)(ka + table_offset_bytes + i * 8);
}

// The four halves of two wave-wide compare masks into lanes LANE (lower half-wave's words) and LANE + 4 (upper half-wave's)
// of `lo` / `hi`: v_writelane_b32 with immediate lane selects. The masks come fresh from vector compares; the idle cycles in
// front give the scalar registers time to land (a v_writelane issued right behind the compare read a stale value on gfx950).
template <int LANE>
__device__ __forceinline__ void write_mask_lanes(uint32_t& lo, uint32_t& hi, uint64_t m0, uint64_t m1) {
    asm volatile("s_nop 4\n\t"
                 "v_writelane_b32 %0, %2, %6\n\t"
                 "v_writelane_b32 %1, %4, %6\n\t"
                 "v_writelane_b32 %0, %3, %7\n\t"
                 "v_writelane_b32 %1, %5, %7"
                 : "+v"(lo), "+v"(hi)
                 : "s"(static_cast<uint32_t>(m0)), "s"(static_cast<uint32_t>(m0 >> 32)), "s"(static_cast<uint32_t>(m1)),
                   "s"(static_cast<uint32_t>(m1 >> 32)), "n"(LANE), "n"(LANE + 4));
}

// The two pointer tables MUST be the first two kernel parameters (offsets 0 and sizeof(StepPtrs)).
// DIRECT (with FAST and STD, no residual): the LIF step runs on the accumulators where the matrix instruction leaves them
// (a lane holds 2 adjacent pixels x 16 channels of the wave's 32 x 64 outputs) and spikes and the membrane go to memory
// from there: the two adjacent pixels of a channel are one 4-byte (spikes) or 8-byte (membrane) store, 32 lanes of a
// half-wave cover a whole 128- or 256-byte line of one channel row. No trip through LDS, and the LIF step does not wait for one.
// BITS_OUT (with DIRECT): the spikes leave row-packed, one byte per 8 pixels of a channel row. The tile's pixel p then sits
// in LDS row p (instead of even pixels in rows 0..31 and odd ones behind them), so that accumulator fragment 0 holds pixels
// 0..31 and fragment 1 pixels 32..63 of the tile: the LIF step's compare masks of the two fragments ARE the 8 bytes of a
// channel row, and a lane per channel stores them. `spikes` then points to bytes, g.spike_step_stride counts bytes, and
// v_out may be null (final membrane not stored).
template <typename XT, int LM, bool STD, int WM, bool FAST, bool DIRECT = false, bool BITS_OUT = false>
__global__ __launch_bounds__(kConvThreads, 2) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_pw_lif_kernel(const StepPtrs xs, const StepPtrs residuals,
                                                                      const int has_residual, const ConvGeom g,
                                                                      const uint16_t* __restrict__ wpacked,
                                                                      const float* __restrict__ bias,
                                                                      const void* __restrict__ v_init,
                                                                      XT* __restrict__ spikes, void* __restrict__ v_out,
                                                                      const LifParams lif) {
    extern __shared__ __align__(16) unsigned char lds[];
    static_assert(!DIRECT || (FAST && STD && sizeof(XT) == 2), "the accumulator-layout LIF step is for the fast variant on 16-bit activations");
    static_assert(!BITS_OUT || DIRECT, "row-packed spikes leave from the accumulator-layout LIF step");
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    constexpr int RPE = (LM == LOAD_PAIR32 || LM == LOAD_ROWBITS) ? 1 : 2;
    static_assert(LM != LOAD_ROWBITS || (FAST && sizeof(XT) == 2), "row-packed spikes: fast variant, 16-bit matrix operands");
    constexpr int SS = kPwSlots;
    constexpr uint32_t ES = static_cast<uint32_t>(sizeof(XT));
    constexpr int NG = 4;                          // epilogue row groups (8 channel rows each) of the wave's 32 channels
    constexpr bool WL = WM == PW_WEIGHTS_LDS;      // weight fragments of the workgroup's 128 channels live in LDS
    constexpr bool WR = WM == PW_WEIGHTS_REGS;     // the wave's weight fragments (exactly 8, one chunk) live in registers
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int l32 = lane & 31;
    const int rg = lane >> 3;                      // epilogue view: channel row inside a group of 8
    const int pcx = lane & 7;                      //                pixels 8 * pcx .. 8 * pcx + 7 of the tile

    const int P = g.W;
    const int groups = 1 << g.groups_log2;
    const int x_buf_bytes = kPwTile * g.pitch;
    const int dbl = g.x_bufs > 1 ? 1 : 0;
    float* __restrict__ stage = reinterpret_cast<float*>(lds + g.x_bufs * x_buf_bytes) + wave * kPwStageFloats;
    unsigned char* __restrict__ wlds = lds + g.x_bufs * x_buf_bytes + kPwStageBytes;
    const int total_pairs = g.nchunks * g.npairs;
    const int nocf = (g.Cout + 31) >> 5;
    const int64_t frag_stride_ocf = static_cast<int64_t>(total_pairs) * (kFragBytes / 2);
    const int steps_with_input = g.shared_x ? 1 : g.T;
    const int64_t row_bytes = LM == LOAD_ROWBITS ? static_cast<int64_t>(P >> 3)   // row-packed spikes: P / 8 bytes per channel row
                                                 : static_cast<int64_t>(P) * ES;  // one channel row of an image

    // ---- kernel constants of the staging: item e = (channel group of 8, pixel pair) of a 64-pixel x CK-channel stage.
    uint32_t item_src[SS], item_dst[SS];
    bool item_on[SS];
#pragma unroll
    for (int s = 0; s < SS; ++s) {
        const int e = s * kConvThreads + tid;
        const int cg = e >> 5, pp = e & 31;
        item_on[s] = cg < groups;
        item_src[s] = LM == LOAD_ROWBITS ? static_cast<uint32_t>(cg) * static_cast<uint32_t>(P) + (static_cast<uint32_t>(pp) >> 2)   // the byte that holds the pair
                                         : (static_cast<uint32_t>(cg) * 8u * static_cast<uint32_t>(P) + 2u * pp) * ES;
        item_dst[s] = static_cast<uint32_t>((BITS_OUT ? 2 * pp : pp) * g.pitch + cg * 16);   // pixel 2 pp -> row pp, pixel 2 pp + 1 -> row pp + 32 (BITS_OUT: rows 2 pp and 2 pp + 1)
    }
    // The 16 bytes of padding behind a pixel's channels are read as a second channel group when a chunk has only one:
    // keep them zero (staging never writes there).
    if (tid < kPwTile * g.x_bufs) {
        const cv_u32x4 zero = {0u, 0u, 0u, 0u};
        *reinterpret_cast<cv_u32x4*>(lds + (tid >> 6) * x_buf_bytes + (tid & 63) * g.pitch + g.CK * 2) = zero;
    }

    // The stage in flight: its data, and which of this thread's items lie outside the image or the channels (bit s).
    uint32_t pre[SS][8][RPE];
    uint32_t pre_bad = 0;
    bool pre_whole = true;

    // Loads of stage (step, chunk) of the tile at pixel px0 of image n. Every load is unconditional: items that lie
    // outside are redirected to the tile's first pixels (always valid) and zeroed on their way into LDS.
    int pre_part = 0;       // fp32 tensors: which of the three parts of the channel axis `pre` holds (2: the low terms)
    auto issue_loads = [&](int step, int chunk, int n, int px0) __attribute__((always_inline)) {
        if constexpr (LM == LOAD_2XF32) split_chunk(chunk, g.nchunks_r, pre_part, chunk);
        const char* __restrict__ base = static_cast<const char*>(kernarg_table_entry(0, step)) +
                                        (LM == LOAD_ROWBITS ? (static_cast<int64_t>(n * g.Cin + chunk * g.CK) * P + px0) >> 3
                                                            : (static_cast<int64_t>(n * g.Cin + chunk * g.CK) * P + px0) * ES);
        const bool whole = (FAST || px0 + kPwTile <= P) && (chunk + 1) * g.CK <= g.Cin;
        uint32_t src[SS], second[SS];
        uint32_t bad = 0;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            src[s] = item_src[s];
            second[s] = ES;
        }
        if (!whole) {
#pragma unroll
            for (int s = 0; s < SS; ++s) {
                const int e = s * kConvThreads + tid;
                const int pix = px0 + 2 * (e & 31);
                const bool ok = chunk * g.CK + (e >> 5) * 8 < g.Cin && (FAST || pix < P);
                src[s] = ok ? item_src[s] : 0u;
                second[s] = (ok && (FAST || pix + 1 < P)) ? ES : 0u;
                bad |= ok ? 0u : (1u << s);
            }
        }
        pre_bad = bad;
        pre_whole = whole;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            if (item_on[s]) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const char* __restrict__ row = base + j * row_bytes;
                    if constexpr (LM == LOAD_PAIR32) {
                        pre[s][j][0] = *reinterpret_cast<const uint32_t*>(row + src[s]);
                    } else if constexpr (LM == LOAD_ROWBITS) {
                        pre[s][j][0] = *reinterpret_cast<const unsigned char*>(row + src[s]);
                    } else if constexpr (LM == LOAD_2X16) {
                        pre[s][j][0] = *reinterpret_cast<const uint16_t*>(row + src[s]);
                        pre[s][j][1] = *reinterpret_cast<const uint16_t*>(row + src[s] + second[s]);
                    } else {
                        pre[s][j][0] = *reinterpret_cast<const uint32_t*>(row + src[s]);
                        pre[s][j][1] = *reinterpret_cast<const uint32_t*>(row + src[s] + second[s]);
                    }
                }
            }
        }
    };

    // Registers -> LDS, transposed to [pixel][channel]: 8 channels of a pixel are one 16-byte write.
    auto write_lds = [&](int buf) __attribute__((always_inline)) {
        unsigned char* __restrict__ xb = lds + buf * x_buf_bytes;
#pragma unroll
        for (int s = 0; s < SS; ++s) {
            if (item_on[s]) {
                cv_u32x4 lo, hi;
                if constexpr (LM == LOAD_ROWBITS) {
                    // The pair's two bits of each channel's byte -> (1.0 or 0, 1.0 or 0) in the matrix operand's 16-bit format.
                    const uint32_t sh = 2u * (static_cast<uint32_t>(tid) & 3u);      // pixel pair pp = tid % 32 sits at bits 2 (pp % 4) of its byte
                    const uint32_t one = F16 ? 0x3C00u : 0x3F80u;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t m = pre[s][j][0] >> sh;
                        pre[s][j][0] = ((m & 1u) ? one : 0u) | ((m & 2u) ? (one << 16) : 0u);
                    }
                }
                if constexpr (LM == LOAD_PAIR32 || LM == LOAD_ROWBITS) {
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
                if (!pre_whole) {
                    const bool zero = (pre_bad >> s) & 1u;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        lo[k] = zero ? 0u : lo[k];
                        hi[k] = zero ? 0u : hi[k];
                    }
                }
                *reinterpret_cast<cv_u32x4*>(xb + item_dst[s]) = lo;
                *reinterpret_cast<cv_u32x4*>(xb + item_dst[s] + (BITS_OUT ? 1 : 32) * g.pitch) = hi;
            }
        }
    };

    // ---- tile walk: pixel tiles congruent to this workgroup's XCD, consecutive work items = output-channel tiles.
    const int xcd = blockIdx.x & 7;
    const int slots_per_xcd = gridDim.x >> 3;
    const int n_px_tiles = g.tiles_x * g.tiles_y;
    const int work_per_xcd = ((n_px_tiles + 7) >> 3) * g.oc_tiles;
    int work = blockIdx.x >> 3;
    int oc_tile = 0, img = 0, px0 = 0;
    auto decode = [&](int w, int& oc_t, int& n, int& p0) __attribute__((always_inline)) -> bool {
        if (w >= work_per_xcd) return false;
        const int pt = fast_div(w, g.d_oc_tiles);
        const int px_tile = pt * 8 + xcd;
        if (px_tile >= n_px_tiles) return false;
        oc_t = w - pt * g.oc_tiles;
        n = fast_div(px_tile, g.d_tiles_x);
        p0 = g.px_base + (px_tile - n * g.tiles_x) * kPwTile;
        return true;
    };
    bool have_tile = decode(work, oc_tile, img, px0);
    if (have_tile) issue_loads(0, 0, img, px0);

    // ---- kernel constants of the matrix loop and the epilogue.
    // This lane's pixels 2 l32 and 2 l32 + 1 sit in rows l32 and l32 + 32 of the tile (consecutive lanes one pitch apart:
    // 16-byte reads without bank conflicts).
    const uint32_t b_off0 = static_cast<uint32_t>(l32 * g.pitch + half * 16);
    const unsigned char* __restrict__ wl = wlds + (static_cast<size_t>(wave) * total_pairs * 64 + lane) * 16;
    // Stage columns are permuted so that both 16-byte reads of a lane's 8 pixels are free of bank conflicts: pixel q sits
    // in column (q & 3) + 4 ((q >> 3) & 7) + 32 ((q >> 2) & 1); a lane's pixel pair stays adjacent.
    float* __restrict__ stage_wr = stage + (half * 4) * kPwStagePitch + 2 * (l32 & 1) + 4 * (l32 >> 2) + 32 * ((l32 >> 1) & 1);
    const float* __restrict__ stage_rd = stage + rg * kPwStagePitch + pcx * 4;
    const float c0f = lif.charge_mode == CHARGE_IF ? 0.0f : 1.0f;
    const float c1f = lif.charge_mode == CHARGE_IF ? 1.0f : lif.inv_tau;
    const bool divide = lif.charge_mode == CHARGE_DIVIDE;   // tau is not a power of two: a true division

    // Bias fragment: row l32 of the weight operand carries the fp32 bias as three 16-bit terms (exact to 24 bits) in its
    // first k-slots; the activation fragments of ones differ in slots the bias fragment leaves zero, only so that the
    // two start-of-timestep matrix instructions stay two instructions.
    cv_u32x4 a_bias = {0u, 0u, 0u, 0u};
    const uint32_t one16 = F16 ? 0x3C00u : 0x3F80u;
    const cv_u32x4 b_ones0 = {one16 | (one16 << 16), one16, 0u, 0u};
    const cv_u32x4 b_ones1 = {one16 | (one16 << 16), one16 | (one16 << 16), 0u, 0u};
    const cv_f32x16 acc_zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    cv_u32x4 a_reg[kPwRegPairs];
    int bias_ocf = -1;
    int loaded_oc_tile = -1;
    int buf = 0;

    while (have_tile) {
        const int ocf = oc_tile * 4 + wave;
        const bool wave_has_work = ocf < nocf;
        const bool full = FAST || px0 + kPwTile <= P;
        const bool fast = FAST || (g.vec8 && full);
        const bool vf32 = FAST || g.v_is_f32;
        uint32_t okmask = 0xffu;
        if (!full) {
            okmask = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) okmask |= (px0 + pcx * 8 + k < P) ? (1u << k) : 0u;
        }
        const int64_t tile_off = static_cast<int64_t>(img) * g.Cout * P + px0;   // uniform element offset into [N, Cout, P]

        if (ocf != bias_ocf) {
            bias_ocf = ocf;
            const int oc = ocf * 32 + l32;
            const float b = (wave_has_work && half == 0 && oc < g.Cout) ? bias[oc] : 0.0f;
            const uint32_t t1 = F16 ? float_to_f16_bits(b) : float_to_bf16_bits(b);
            const float r1 = b - (F16 ? f16_bits_to_float(t1) : bf16_bits_to_float(t1));
            const uint32_t t2 = F16 ? float_to_f16_bits(r1) : float_to_bf16_bits(r1);
            const float r2 = r1 - (F16 ? f16_bits_to_float(t2) : bf16_bits_to_float(t2));
            const uint32_t t3 = F16 ? float_to_f16_bits(r2) : float_to_bf16_bits(r2);
            a_bias[0] = t1 | (t2 << 16);
            a_bias[1] = t3;
        }
        if (WR && ocf != loaded_oc_tile) {
            loaded_oc_tile = ocf;
            const uint16_t* __restrict__ src = wpacked + static_cast<int64_t>(min(ocf, nocf - 1)) * frag_stride_ocf + lane * 8;
#pragma unroll
            for (int q = 0; q < kPwRegPairs; ++q)
                a_reg[q] = *reinterpret_cast<const cv_u32x4*>(src + q * (kFragBytes / 2));
            // Wait here, once: otherwise every later use of a fragment waits for ALL outstanding loads, prefetch included.
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        }
        if (WL && oc_tile != loaded_oc_tile) {
            // (Re)load the weight fragments of this output-channel tile: [wave][pair][lane] x 16 bytes.
            __syncthreads();
            const int vec_per_wave = total_pairs * 64;
            for (int i = tid; i < 4 * vec_per_wave; i += kConvThreads) {
                const int wv = i / vec_per_wave;
                const int within = i - wv * vec_per_wave;
                const int src_ocf = min(oc_tile * 4 + wv, nocf - 1);
                const cv_u32x4 val = *reinterpret_cast<const cv_u32x4*>(wpacked + static_cast<int64_t>(src_ocf) * frag_stride_ocf + static_cast<int64_t>(within) * 8);
                *reinterpret_cast<cv_u32x4*>(wlds + static_cast<size_t>(i) * 16) = val;
            }
            loaded_oc_tile = oc_tile;
            __syncthreads();
        }
        const uint16_t* __restrict__ wg = wpacked + static_cast<int64_t>(min(ocf, nocf - 1)) * frag_stride_ocf + lane * 8;

        // ---- membrane of this lane's 4 x 8 neurons (group gi: channel ocf * 32 + gi * 8 + rg, pixels 8 pcx ..), all T steps.
        uint32_t lane_off[NG];   // bytes into a spike-typed [Cout, P] image
        bool row_ok[NG];
        float v[NG][8];
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            const int oc = ocf * 32 + gi * 8 + rg;
            row_ok[gi] = FAST ? wave_has_work : (wave_has_work && oc < g.Cout && okmask != 0);
            lane_off[gi] = static_cast<uint32_t>(oc * P + pcx * 8) * ES;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[gi][k] = 0.0f;
        }
        // DIRECT: membrane of the lane's 2 pixels x 16 channels, register r = channel ocf * 32 + 8 (r / 4) + 4 half + r % 4.
        float vd[kNPF][16];
        const uint32_t lane_off_d = static_cast<uint32_t>((ocf * 32 + 4 * half) * P + (BITS_OUT ? l32 : 2 * l32));   // elements into [Cout, P]
        auto row_off_d = [&](int r) __attribute__((always_inline)) { return static_cast<uint32_t>((8 * (r >> 2) + (r & 3)) * P); };
        if constexpr (DIRECT) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                vd[0][r] = 0.0f;
                vd[1][r] = 0.0f;
            }
            if (v_init != nullptr && wave_has_work) {
                const float* __restrict__ vsrc = static_cast<const float*>(v_init) + tile_off + lane_off_d;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if constexpr (BITS_OUT) {      // the lane's pixels are l32 and l32 + 32 of the tile
                        vd[0][r] = vsrc[row_off_d(r)];
                        vd[1][r] = vsrc[row_off_d(r) + 32];
                    } else {
                        const Pack<float, 2> two = *reinterpret_cast<const Pack<float, 2>*>(vsrc + row_off_d(r));
                        vd[0][r] = two.v[0];
                        vd[1][r] = two.v[1];
                    }
                }
            }
        }
        if (!DIRECT && v_init != nullptr) {
            if (fast && vf32) {
                const char* vbase = reinterpret_cast<const char*>(static_cast<const float*>(v_init) + tile_off);
#pragma unroll
                for (int gi = 0; gi < NG; ++gi) {
                    if (row_ok[gi]) {
                        const float* src = reinterpret_cast<const float*>(vbase + lane_off[gi] * (4u / ES));
                        const Pack<float, 4> lo = *reinterpret_cast<const Pack<float, 4>*>(src);
                        const Pack<float, 4> hi = *reinterpret_cast<const Pack<float, 4>*>(src + 4);
#pragma unroll
                        for (int k = 0; k < 4; ++k) { v[gi][k] = lo.v[k]; v[gi][4 + k] = hi.v[k]; }
                    }
                }
            } else {
#pragma unroll
                for (int gi = 0; gi < NG; ++gi) {
                    if (row_ok[gi]) {
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            if (okmask & (1u << k)) {
                                v[gi][k] = vf32 ? static_cast<const float*>(v_init)[tile_off + lane_off[gi] / ES + k]
                                                      : to_float(static_cast<const XT*>(v_init)[tile_off + lane_off[gi] / ES + k]);
                            }
                        }
                    }
                }
            }
        }

        // Spikes of a timestep wait here until the next stage has left its load registers.
        Pack<XT, 8> pend[NG];
        uint32_t pend_d[16];     // DIRECT: the spikes of 2 adjacent pixels of channel register r
        uint32_t pend_lo = 0u, pend_hi = 0u;   // BITS_OUT: lane c < 32 holds the tile's 64 spike bits of channel ocf * 32 + c
        int pend_step = -1;
        auto flush_spikes = [&]() __attribute__((always_inline)) {
            char* __restrict__ out = reinterpret_cast<char*>(spikes + pend_step * g.spike_step_stride + tile_off);
            if constexpr (BITS_OUT) {
                unsigned char* __restrict__ row = reinterpret_cast<unsigned char*>(spikes) + pend_step * g.spike_step_stride +
                                                  ((tile_off + static_cast<int64_t>(ocf) * 32 * P) >> 3);
                const snnf_u32x2 word = {pend_lo, pend_hi};
                if (lane < 32) *reinterpret_cast<snnf_u32x2*>(row + static_cast<uint32_t>(lane) * static_cast<uint32_t>(P >> 3)) = word;
            } else if constexpr (DIRECT) {
                // Uniform row base + 32-bit lane offset: the stores take the scalar-base addressing form.
                const uint32_t lane_b = lane_off_d * ES;
                if (g.stream_out) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        Pack<XT, 2> two;
                        *reinterpret_cast<uint32_t*>(&two) = pend_d[r];
                        store_streaming(reinterpret_cast<XT*>(out + static_cast<size_t>(row_off_d(r)) * ES + lane_b), two);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) *reinterpret_cast<uint32_t*>(out + static_cast<size_t>(row_off_d(r)) * ES + lane_b) = pend_d[r];
                }
            } else if (fast) {
#pragma unroll
                for (int gi = 0; gi < NG; ++gi)
                    if (row_ok[gi]) {
                        if (g.stream_out) store_streaming(reinterpret_cast<XT*>(out + lane_off[gi]), pend[gi]);
                        else *reinterpret_cast<Pack<XT, 8>*>(out + lane_off[gi]) = pend[gi];
                    }
            } else {
#pragma unroll
                for (int gi = 0; gi < NG; ++gi) {
                    if (row_ok[gi]) {
#pragma unroll
                        for (int k = 0; k < 8; ++k)
                            if (okmask & (1u << k)) *reinterpret_cast<XT*>(out + lane_off[gi] + k * ES) = pend[gi].v[k];
                    }
                }
            }
            pend_step = -1;
        };

        cv_f32x16 acc[kNPF];
        int next_work = work, next_oc_tile = oc_tile, next_img = img, next_px0 = px0;
        bool next_tile = false;
        for (int step = 0; step < g.T; ++step) {
            if (step < steps_with_input) {
                acc[0] = cv_mfma<F16>(a_bias, b_ones0, acc_zero);
                acc[1] = cv_mfma<F16>(a_bias, b_ones1, acc_zero);
                for (int chunk = 0; chunk < g.nchunks; ++chunk) {
                    if (!dbl) __syncthreads();   // single buffer: every wave is done reading the previous stage
                    write_lds(buf);              // waits for the stage's loads
                    __syncthreads();
                    if (pend_step >= 0) flush_spikes();
                    // ---- the stage after this one: next chunk, next timestep, or the first stage of the next tile.
                    int ns = step, nc = chunk + 1, nimg = img, npx = px0;
                    bool more = true;
                    if (nc == g.nchunks) {
                        nc = 0;
                        ns = step + 1;
                        if (ns == steps_with_input) {
                            ns = 0;
                            next_work = work + slots_per_xcd;
                            next_tile = decode(next_work, next_oc_tile, next_img, next_px0);
                            more = next_tile;
                            nimg = next_img;
                            npx = next_px0;
                        }
                    }
                    if (WM != PW_WEIGHTS_STREAM && more) issue_loads(ns, nc, nimg, npx);
                    if (wave_has_work) {
                        const unsigned char* __restrict__ bp0 = lds + buf * x_buf_bytes + b_off0;
                        const unsigned char* __restrict__ bp1 = bp0 + 32 * g.pitch;
                        int pair = 0;
                        if constexpr (WR) {
                            // Exactly kPwRegPairs pairs, straight-line: operand reads run two pairs ahead of the matrix unit.
                            cv_u32x4 b0[kPwRegPairs], b1[kPwRegPairs];
#pragma unroll
                            for (int q = 0; q < kPwRegPairs; ++q) {
                                b0[q] = *reinterpret_cast<const cv_u32x4*>(bp0 + q * 32);
                                b1[q] = *reinterpret_cast<const cv_u32x4*>(bp1 + q * 32);
                            }
#pragma unroll
                            for (int q = 0; q < kPwRegPairs; ++q) {
                                acc[0] = cv_mfma<F16>(a_reg[q], b0[q], acc[0]);
                                acc[1] = cv_mfma<F16>(a_reg[q], b1[q], acc[1]);
                            }
                            __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
                            for (int q = 0; q < kPwRegPairs - 2; ++q) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                            }
                            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                        } else if constexpr (WL) {
                            const unsigned char* __restrict__ ap = wl + static_cast<size_t>(chunk * g.npairs) * kFragBytes;
                            for (; pair + 4 <= g.npairs; pair += 4) {
                                // All twelve operand reads go out before the first matrix instruction.
                                cv_u32x4 a[4], b0[4], b1[4];
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    a[q] = *reinterpret_cast<const cv_u32x4*>(ap + (pair + q) * kFragBytes);
                                    b0[q] = *reinterpret_cast<const cv_u32x4*>(bp0 + (pair + q) * 32);
                                    b1[q] = *reinterpret_cast<const cv_u32x4*>(bp1 + (pair + q) * 32);
                                }
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    acc[0] = cv_mfma<F16>(a[q], b0[q], acc[0]);
                                    acc[1] = cv_mfma<F16>(a[q], b1[q], acc[1]);
                                }
                                // Instruction order for the scheduler: two pairs' operands in flight ahead of the matrix unit.
                                __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
                                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                            }
                            for (; pair + 2 <= g.npairs; pair += 2) {
                                const cv_u32x4 a0 = *reinterpret_cast<const cv_u32x4*>(ap + pair * kFragBytes);
                                const cv_u32x4 a1 = *reinterpret_cast<const cv_u32x4*>(ap + (pair + 1) * kFragBytes);
                                const cv_u32x4 b00 = *reinterpret_cast<const cv_u32x4*>(bp0 + pair * 32);
                                const cv_u32x4 b01 = *reinterpret_cast<const cv_u32x4*>(bp1 + pair * 32);
                                const cv_u32x4 b10 = *reinterpret_cast<const cv_u32x4*>(bp0 + pair * 32 + 32);
                                const cv_u32x4 b11 = *reinterpret_cast<const cv_u32x4*>(bp1 + pair * 32 + 32);
                                acc[0] = cv_mfma<F16>(a0, b00, acc[0]);
                                acc[1] = cv_mfma<F16>(a0, b01, acc[1]);
                                acc[0] = cv_mfma<F16>(a1, b10, acc[0]);
                                acc[1] = cv_mfma<F16>(a1, b11, acc[1]);
                            }
                            if (pair < g.npairs) {
                                const cv_u32x4 a0 = *reinterpret_cast<const cv_u32x4*>(ap + pair * kFragBytes);
                                const cv_u32x4 b00 = *reinterpret_cast<const cv_u32x4*>(bp0 + pair * 32);
                                const cv_u32x4 b01 = *reinterpret_cast<const cv_u32x4*>(bp1 + pair * 32);
                                acc[0] = cv_mfma<F16>(a0, b00, acc[0]);
                                acc[1] = cv_mfma<F16>(a0, b01, acc[1]);
                            }
                        } else {
                            // Weights streamed from global memory (L2 resident), one fragment ahead.
                            const uint16_t* __restrict__ ap = wg + static_cast<int64_t>(chunk * g.npairs) * (kFragBytes / 2);
                            cv_u32x4 a_cur = *reinterpret_cast<const cv_u32x4*>(ap);
                            for (; pair < g.npairs; ++pair) {
                                const int pn = pair + 1 < g.npairs ? pair + 1 : pair;
                                const cv_u32x4 a_nxt = *reinterpret_cast<const cv_u32x4*>(ap + pn * (kFragBytes / 2));
                                const cv_u32x4 b0 = *reinterpret_cast<const cv_u32x4*>(bp0 + pair * 32);
                                const cv_u32x4 b1 = *reinterpret_cast<const cv_u32x4*>(bp1 + pair * 32);
                                acc[0] = cv_mfma<F16>(a_cur, b0, acc[0]);
                                acc[1] = cv_mfma<F16>(a_cur, b1, acc[1]);
                                a_cur = a_nxt;
                            }
                        }
                    }
                    // Streaming weights share the load counter: the next stage's loads go out behind them.
                    if (WM == PW_WEIGHTS_STREAM && more) issue_loads(ns, nc, nimg, npx);
                    buf ^= dbl;
                }
            }

            // ---- LIF step: 8 channel rows at a time through the wave's stage, so that a lane owns 8 consecutive pixels.
            if (wave_has_work) {
                if (pend_step >= 0) flush_spikes();   // only when a timestep had no stage of its own (shared frame)
                const char* __restrict__ res_t =
                    has_residual ? reinterpret_cast<const char*>(static_cast<const XT*>(kernarg_table_entry(sizeof(StepPtrs), step)) + tile_off) : nullptr;
                if constexpr (BITS_OUT) {
                    // The compare of the LIF step is the ballot: bits 0..31 of a mask are the lower half-wave's channel row
                    // (8 (r / 4) + r % 4), bits 32..63 the upper one's (4 rows on), for pixels 0..31 (fragment 0) or 32..63.
                    // (the lane selects of v_writelane are immediates: one macro expansion per register)
#define SNNF_PW_BITS_ROW(r)                                                                                                  \
    {                                                                                                                        \
        const float h0 = vd[0][r] + (acc[0][r] - vd[0][r]) * lif.inv_tau;                                                    \
        const float h1 = vd[1][r] + (acc[1][r] - vd[1][r]) * lif.inv_tau;                                                    \
        const bool f0 = h0 >= lif.v_threshold;                                                                               \
        const bool f1 = h1 >= lif.v_threshold;                                                                               \
        vd[0][r] = f0 ? lif.v_reset : h0;                                                                                    \
        vd[1][r] = f1 ? lif.v_reset : h1;                                                                                    \
        const uint64_t m0 = __builtin_amdgcn_ballot_w64(f0);                                                                 \
        const uint64_t m1 = __builtin_amdgcn_ballot_w64(f1);                                                                 \
        write_mask_lanes<8 * ((r) >> 2) + ((r) & 3)>(pend_lo, pend_hi, m0, m1);                                              \
    }
                    SNNF_PW_BITS_ROW(0) SNNF_PW_BITS_ROW(1) SNNF_PW_BITS_ROW(2) SNNF_PW_BITS_ROW(3)
                    SNNF_PW_BITS_ROW(4) SNNF_PW_BITS_ROW(5) SNNF_PW_BITS_ROW(6) SNNF_PW_BITS_ROW(7)
                    SNNF_PW_BITS_ROW(8) SNNF_PW_BITS_ROW(9) SNNF_PW_BITS_ROW(10) SNNF_PW_BITS_ROW(11)
                    SNNF_PW_BITS_ROW(12) SNNF_PW_BITS_ROW(13) SNNF_PW_BITS_ROW(14) SNNF_PW_BITS_ROW(15)
#undef SNNF_PW_BITS_ROW
                } else if constexpr (DIRECT) {
                    const uint32_t one16 = F16 ? 0x3C00u : 0x3F80u;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        uint32_t pair = 0u;
#pragma unroll
                        for (int pf = 0; pf < kNPF; ++pf) {
                            const float h = vd[pf][r] + (acc[pf][r] - vd[pf][r]) * lif.inv_tau;
                            const bool fired = h >= lif.v_threshold;
                            vd[pf][r] = fired ? lif.v_reset : h;
                            pair |= fired ? (one16 << (16 * pf)) : 0u;
                        }
                        pend_d[r] = pair;
                    }
                }
#pragma unroll
                for (int gi = 0; gi < (DIRECT ? 0 : NG); ++gi) {
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const cv_f32x2 two = {acc[0][gi * 4 + rr], acc[1][gi * 4 + rr]};
                        *reinterpret_cast<cv_f32x2*>(stage_wr + rr * kPwStagePitch) = two;
                    }
                    __builtin_amdgcn_wave_barrier();
                    const Pack<float, 4> xlo = *reinterpret_cast<const Pack<float, 4>*>(stage_rd);
                    const Pack<float, 4> xhi = *reinterpret_cast<const Pack<float, 4>*>(stage_rd + 32);
                    float x[8];
#pragma unroll
                    for (int k = 0; k < 4; ++k) { x[k] = xlo.v[k]; x[4 + k] = xhi.v[k]; }
                    if (res_t != nullptr && row_ok[gi]) {
                        if (fast) {
                            const Pack<XT, 8> rr8 = *reinterpret_cast<const Pack<XT, 8>*>(res_t + lane_off[gi]);
#pragma unroll
                            for (int k = 0; k < 8; ++k) x[k] += to_float(rr8.v[k]);
                        } else {
#pragma unroll
                            for (int k = 0; k < 8; ++k)
                                if (okmask & (1u << k)) x[k] += to_float(*reinterpret_cast<const XT*>(res_t + lane_off[gi] + k * ES));
                        }
                    }
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
                        pend[gi].v[k] = spike_value<XT>(fired);
                    }
                }
                pend_step = step;
            }
        }

        // ---- last timestep's spikes and the final membrane.
        if (pend_step >= 0) flush_spikes();
        if constexpr (BITS_OUT) {
            if (wave_has_work && v_out != nullptr) {
                float* __restrict__ vdst = static_cast<float*>(v_out) + tile_off + lane_off_d;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    vdst[row_off_d(r)] = vd[0][r];
                    vdst[row_off_d(r) + 32] = vd[1][r];
                }
            }
        } else if constexpr (DIRECT) {
            if (wave_has_work) {
                char* __restrict__ vbase = reinterpret_cast<char*>(static_cast<float*>(v_out) + tile_off);   // uniform
                const uint32_t lane_vb = lane_off_d * 4u;
                if (g.stream_out) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const Pack<float, 2> two = {{vd[0][r], vd[1][r]}};
                        store_streaming(reinterpret_cast<float*>(vbase + static_cast<size_t>(row_off_d(r)) * 4u + lane_vb), two);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const Pack<float, 2> two = {{vd[0][r], vd[1][r]}};
                        *reinterpret_cast<Pack<float, 2>*>(vbase + static_cast<size_t>(row_off_d(r)) * 4u + lane_vb) = two;
                    }
                }
            }
        } else if (fast && vf32) {
            char* vbase = reinterpret_cast<char*>(static_cast<float*>(v_out) + tile_off);
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                if (row_ok[gi]) {
                    float* dst = reinterpret_cast<float*>(vbase + lane_off[gi] * (4u / ES));
                    Pack<float, 4> lo, hi;
#pragma unroll
                    for (int k = 0; k < 4; ++k) { lo.v[k] = v[gi][k]; hi.v[k] = v[gi][4 + k]; }
                    if (g.stream_out) {
                        store_streaming(dst, lo);
                        store_streaming(dst + 4, hi);
                    } else {
                        *reinterpret_cast<Pack<float, 4>*>(dst) = lo;
                        *reinterpret_cast<Pack<float, 4>*>(dst + 4) = hi;
                    }
                }
            }
        } else {
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                if (row_ok[gi]) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        if (okmask & (1u << k)) {
                            if (vf32) static_cast<float*>(v_out)[tile_off + lane_off[gi] / ES + k] = v[gi][k];
                            else static_cast<XT*>(v_out)[tile_off + lane_off[gi] / ES + k] = from_float<XT>(v[gi][k]);
                        }
                    }
                }
            }
        }
        work = next_work;
        oc_tile = next_oc_tile;
        img = next_img;
        px0 = next_px0;
        have_tile = next_tile;
    }
}

template <typename XT>
int launch_conv_pw(const ConvLaunch& L, int load_mode, bool fast) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kConvThreads, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.has_residual, L.g, L.wpacked, L.bias, L.v_init,
                                                                      static_cast<XT*>(L.spikes), L.v_out, L.lif);
        return check_launch("snnf_conv_lif");
    };
    // Fast variants exist for the common neuron only (power-of-two tau, hard reset); the general variants take any
    // neuron through the generic update and keep their weights in LDS or stream them.
    auto pick = [&](auto lm) -> int {
        constexpr int LMV = decltype(lm)::value;
        if constexpr (sizeof(XT) == 2) {
            if (fast && !L.has_residual) {      // LIF on the accumulators (16-bit spikes: two pixels are one 4-byte store)
                if (L.g.w_lds == PW_WEIGHTS_REGS) return run(conv_pw_lif_kernel<XT, LMV, true, PW_WEIGHTS_REGS, true, true>);
                if (L.g.w_lds == PW_WEIGHTS_LDS) return run(conv_pw_lif_kernel<XT, LMV, true, PW_WEIGHTS_LDS, true, true>);
                return run(conv_pw_lif_kernel<XT, LMV, true, PW_WEIGHTS_STREAM, true, true>);
            }
        }
        if (fast) {
            if (L.g.w_lds == PW_WEIGHTS_REGS) return run(conv_pw_lif_kernel<XT, LMV, true, PW_WEIGHTS_REGS, true>);
            if (L.g.w_lds == PW_WEIGHTS_LDS) return run(conv_pw_lif_kernel<XT, LMV, true, PW_WEIGHTS_LDS, true>);
            return run(conv_pw_lif_kernel<XT, LMV, true, PW_WEIGHTS_STREAM, true>);
        }
        if (L.g.w_lds == PW_WEIGHTS_LDS) return run(conv_pw_lif_kernel<XT, LMV, false, PW_WEIGHTS_LDS, false>);
        return run(conv_pw_lif_kernel<XT, LMV, false, PW_WEIGHTS_STREAM, false>);
    };
    if constexpr (sizeof(XT) == 4) {
        return pick(std::integral_constant<int, LOAD_2XF32>{});
    } else {
        if (load_mode == LOAD_ROWBITS) {    // row-packed spikes in: the fast variants with the LIF step on the accumulators
            if (!fast || L.has_residual) return fail(SNNF_ERR_UNSUPPORTED, "snnf_pwconv_lif_rowbits: unsupported_shape: only layers the fast variant takes");
            if (L.g.bits_out) {
                if (L.g.w_lds == PW_WEIGHTS_REGS) return run(conv_pw_lif_kernel<XT, LOAD_ROWBITS, true, PW_WEIGHTS_REGS, true, true, true>);
                if (L.g.w_lds == PW_WEIGHTS_LDS) return run(conv_pw_lif_kernel<XT, LOAD_ROWBITS, true, PW_WEIGHTS_LDS, true, true, true>);
                return run(conv_pw_lif_kernel<XT, LOAD_ROWBITS, true, PW_WEIGHTS_STREAM, true, true, true>);
            }
            if (L.g.w_lds == PW_WEIGHTS_REGS) return run(conv_pw_lif_kernel<XT, LOAD_ROWBITS, true, PW_WEIGHTS_REGS, true, true>);
            if (L.g.w_lds == PW_WEIGHTS_LDS) return run(conv_pw_lif_kernel<XT, LOAD_ROWBITS, true, PW_WEIGHTS_LDS, true, true>);
            return run(conv_pw_lif_kernel<XT, LOAD_ROWBITS, true, PW_WEIGHTS_STREAM, true, true>);
        }
        if (load_mode == LOAD_PAIR32) return pick(std::integral_constant<int, LOAD_PAIR32>{});
        return pick(std::integral_constant<int, LOAD_2X16>{});
    }
}

}  // namespace snnf
