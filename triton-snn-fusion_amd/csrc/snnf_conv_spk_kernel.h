// Dense convolution + bias (+ residual) + LIF on activations in the library's internal layouts: channel-blocked 16-bit
// values ([N][C/8][H][W][8], "C8") or bit-packed spikes ([N][C/8][H][W] bytes, bit j = channel 8 c8 + j, "BITS"). These
// layouts exist between consecutive fused operators of one network; the operator boundary keeps dense NCHW.
//
// Same implicit GEMM as the NCHW kernels (M = output channels from packed weight fragments, N = pixels, K = taps x
// channel groups of 8, v_mfma_f32_32x32x16, fp32 accumulate, TT timesteps side by side against one weight fragment), but:
//   * a group of 8 channels of one pixel is 16 contiguous bytes in C8 and one byte in BITS, i.e. already the matrix
//     operand of a lane: staging is one load and one 16-byte LDS write per item, no transposition; a spike byte is
//     expanded to eight 16-bit ones with 13 integer instructions on its way into LDS;
//   * every wave is its own pipeline: it owns a patch of 32 output pixels x 64 output channels x TT timesteps, stages
//     the halo of its patch into a private LDS region and never meets a workgroup barrier in the matrix loop, so the
//     eight waves of a compute unit drift apart and one wave's staging and epilogue overlap another's matrix work;
//   * spikes leave as bits: the accumulator layout gives a lane 4 consecutive channels of its pixel, the two halves of
//     a wave exchange their nibbles with one cross-lane move and store bytes; the membrane is fp32 NCHW and optional;
//   * deep layers with few pixels split K over WK waves of a workgroup (whole LDS stages each) and add their partial
//     sums through LDS in a fixed order, one timestep per round.
#pragma once

#include <type_traits>

#include "snnf_conv_common.h"

namespace snnf {

typedef __bf16 sk_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 sk_f16x8 __attribute__((ext_vector_type(8)));
typedef float sk_f32x16 __attribute__((ext_vector_type(16)));
typedef float sk_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kSpkWaves = 8;                      // waves per workgroup, one workgroup per compute unit
#ifndef SPK_SLOTS
#define SPK_SLOTS 8
#endif
constexpr int kSpkSlots = SPK_SLOTS;                      // staging items per lane and timestep, at most
constexpr size_t kSpkPartialBytes = kSpkWaves * 8 * 64 * 16;   // split-K: one timestep's partial sums of all waves

struct SpkGeom {
    int N, Cin, H, W, Cout, KH, KW, sh, sw, ph, pw, Ho, Wo;
    int C8in, C8out;
    int PR, PC, PI;              // patch of a wave: PR x PC output pixels of PI images (PI > 1: whole planes)
    int patches_x, patches_img;  // patches per output row band, per image (patches_x * patches_y)
    int n_patches;               // image groups x patches per image
    int RR, RC;                  // halo rows / columns per image
    int region;                  // PI * RR * RC: 16-byte items per channel group and timestep
    int G;                       // channel groups per LDS stage
    int nstages;                 // ceil(C8in / G)
    int IT, JT;                  // staging items per timestep (G * region) and slots per lane (ceil(IT / 64))
    int gpc;                     // channel groups per packed chunk (CK / 8)
    int npairs;                  // k-slot pairs per packed chunk
    int nocf;                    // 32-row weight fragments
    int tap_pairs;               // packed chunks of 8 channels: a pair of k-slots is two taps of one group
    int taps;
    int T;                       // timesteps
    int shared_x;                // one input frame for all T timesteps (TT == 1): convolved once
    int wk_log2;                 // split-K: waves per tile
    int n_items, iters;          // (patch, 64-channel tile) pairs; loop trips per wave
    int in_layout, res_layout, out_layout;   // snnf_layout codes; res_layout < 0: no residual
    int analog_out;              // no neuron: the sums themselves are written (C8 or NCHW)
    int64_t out_step_stride;     // bytes between timesteps of `out`
    int lds_wave_bytes;          // private staging region of a wave (a multiple of 16)
    int64_t frag_stride;         // 16-bit elements between consecutive 32-row fragments of the packed weight
    FastDiv d_ppx, d_PC, d_region, d_rrrc, d_RC, d_n_patches, d_patches_img, d_patches_x, d_gpc, d_hg, d_nst, d_KW;
};

struct SpkLaunch {
    StepPtrs xs;
    StepPtrs residuals;
    SpkGeom g;
    const uint16_t* wpacked;
    const float* bias;
    const float* v_init;
    void* out;
    float* v_out;
    LifParams lif;
    int grid;
    size_t lds_bytes;
    hipStream_t stream;
};

template <bool F16>
__device__ __forceinline__ sk_f32x16 sk_mfma(sk_u32x4 a, sk_u32x4 b, sk_f32x16 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(sk_f16x8, a), __builtin_bit_cast(sk_f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(sk_bf16x8, a), __builtin_bit_cast(sk_bf16x8, b), c, 0, 0, 0);
    }
}

// Entry i of a table of pointers passed by value as a kernel argument, read from the kernel-argument segment (arguments
// start at offset 0 of that segment, in declaration order and naturally aligned): indexing the by-value struct with a
// runtime index would copy it to scratch memory.
typedef const void* sk_cvp;
__device__ __forceinline__ const void* sk_kernarg_ptr(int table_offset_bytes, int i) {
    typedef const __attribute__((address_space(4))) unsigned char* ka_bytes;
    typedef const __attribute__((address_space(4))) sk_cvp* ka_entry;
    ka_bytes ka = (ka_bytes)__builtin_amdgcn_kernarg_segment_ptr();
    return *(ka_entry)(ka + table_offset_bytes + i * 8);
}

// Eight spike bits -> eight 16-bit ones or zeros (ONE = the dtype's 1.0), channel j in element j.
template <uint32_t ONE>
__device__ __forceinline__ sk_u32x4 sk_expand_bits(uint32_t byte) {
    const uint32_t m = __umul24(byte, 0x8001u);   // bit i of the byte at bits i and 15 + i
    sk_u32x4 d;
    d[0] = __umul24(m & 0x10001u, ONE);
    d[1] = __umul24((m >> 2) & 0x10001u, ONE);
    d[2] = __umul24((m >> 4) & 0x10001u, ONE);
    d[3] = __umul24((m >> 6) & 0x10001u, ONE);
    return d;
}

template <typename XT, int TT, int IN, bool SK>
__global__ __launch_bounds__(kSpkWaves * 64, 1) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_spk_kernel(
    const StepPtrs xs, const StepPtrs residuals, const SpkGeom g, const uint16_t* __restrict__ wpacked,
    const float* __restrict__ bias, const float* __restrict__ v_init, unsigned char* __restrict__ out,
    float* __restrict__ v_out, const LifParams lif) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    constexpr uint32_t ONE = F16 ? 0x3c00u : 0x3f80u;
    constexpr int kResTable = static_cast<int>(sizeof(StepPtrs));
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int l32 = lane & 31;
    unsigned char* const wlds = lds + wave * g.lds_wave_bytes;
    const int region16 = g.region * 16;        // bytes of one channel group of the halo
    const int tile_t = g.G * region16;         // bytes of one timestep's stage

    // ---- this lane's output pixel inside the patch, and where its top-left input sits in the staged halo.
    const int ppx = g.PR * g.PC;
    const int pi = fast_div(l32, g.d_ppx);
    const int prem = l32 - pi * ppx;
    const int prow = fast_div(prem, g.d_PC);
    const int pcol = prem - prow * g.PC;
    const bool lane_in_patch = pi < g.PI;
    const uint32_t lane_b = lane_in_patch ? static_cast<uint32_t>(((pi * g.RR + prow * g.sh) * g.RC + pcol * g.sw) * 16) : 0u;

    const int WK = SK ? (1 << g.wk_log2) : 1;
    const int wk = SK ? (wave & (WK - 1)) : 0;
    const int tile_in_block = SK ? (wave >> g.wk_log2) : wave;
    const int tiles_per_block = SK ? (kSpkWaves >> g.wk_log2) : kSpkWaves;
    const int po = g.Ho * g.Wo;
    const int nsteps_t = g.shared_x ? 1 : g.T;          // timesteps with a convolution of their own
    const uint16_t* __restrict__ wlane = wpacked + lane * 8;
    const int hg = g.tap_pairs ? 1 : (g.G >> 1);        // k-slot pairs per tap and stage
    const int nst = g.tap_pairs ? g.npairs : g.taps * hg;   // matrix steps per stage

    for (int it = 0; it < g.iters; ++it) {
        // Consecutive items go to consecutive workgroups, so that a layer with fewer items than wave slots still uses every compute unit.
        const int item = (it * tiles_per_block + tile_in_block) * static_cast<int>(gridDim.x) + static_cast<int>(blockIdx.x);
        const bool have = item < g.n_items;
        const int item_c = have ? item : 0;
        const int oc_tile = fast_div(item_c, g.d_n_patches);
        const int patch = item_c - oc_tile * g.n_patches;
        const int imgg = fast_div(patch, g.d_patches_img);
        const int prem_i = patch - imgg * g.patches_img;
        const int py = fast_div(prem_i, g.d_patches_x);
        const int n0 = imgg * g.PI;
        const int oh0 = py * g.PR;
        const int ow0 = (prem_i - py * g.patches_x) * g.PC;
        const int ih_lo = oh0 * g.sh - g.ph;
        const int iw_lo = ow0 * g.sw - g.pw;

        const int ocf0 = oc_tile * 2;
        const int64_t w_off0 = static_cast<int64_t>(min(ocf0, g.nocf - 1)) * g.frag_stride;
        const int64_t w_off1 = static_cast<int64_t>(min(ocf0 + 1, g.nocf - 1)) * g.frag_stride;

        // ---- this lane's output pixel.
        const int n = n0 + pi;
        const int oh = oh0 + prow;
        const int ow = ow0 + pcol;
        const bool px_ok = have && lane_in_patch && n < g.N && oh < g.Ho && ow < g.Wo;
        const int pxo = px_ok ? oh * g.Wo + ow : 0;
        const int n_c = px_ok ? n : 0;

        for (int t0 = 0; t0 < nsteps_t; t0 += TT) {
            sk_f32x16 acc[TT][2];
#pragma unroll
            for (int t = 0; t < TT; ++t)
#pragma unroll
                for (int f = 0; f < 2; ++f)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[t][f][r] = 0.0f;

            // One LDS stage: G channel groups of the patch's halo for TT timesteps, from global memory into this wave's region.
            // Item e = slot * 64 + lane of a timestep = (group, image, row, column) of the halo; its LDS address is 16 e. Items
            // are decoded on the fly (nothing about them is kept in registers across the matrix loop) and move in batches of 4
            // slots x TT timesteps: all loads of a batch are in flight together.
            auto stage_in = [&](int s) __attribute__((always_inline)) {
                const int gg0 = s * g.G;
                const int base_u = ((n0 * g.C8in + gg0) * g.H + ih_lo) * g.W + iw_lo;   // may be negative; only added to in-image items
                __builtin_amdgcn_wave_barrier();   // the matrix steps of the previous stage have read their operands
#pragma unroll
                for (int jb = 0; jb < kSpkSlots; jb += 4) {
                    if (jb < g.JT) {
                        int idx[4];
                        uint32_t ok_bits = 0;       // bit j: the item is real data; bit 4 + j: the item exists (is written)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int e = (jb + j) * 64 + lane;
                            const int gq = fast_div(e, g.d_region);
                            const int rem = e - gq * g.region;
                            const int ii = fast_div(rem, g.d_rrrc);
                            const int rem2 = rem - ii * (g.RR * g.RC);
                            const int r = fast_div(rem2, g.d_RC);
                            const int c = rem2 - r * g.RC;
                            const int ih = ih_lo + r, iw = iw_lo + c;
                            const bool exists = e < g.IT;
                            const bool ok = exists && n0 + ii < g.N && gg0 + gq < g.C8in && static_cast<unsigned>(ih) < static_cast<unsigned>(g.H) &&
                                            static_cast<unsigned>(iw) < static_cast<unsigned>(g.W);
                            idx[j] = ok ? base_u + ((ii * g.C8in + gq) * g.H + r) * g.W + c : 0;
                            ok_bits |= (ok ? (1u << j) : 0u) | (exists ? (16u << j) : 0u);
                        }
                        if constexpr (IN == SNNF_LAYOUT_BITS) {
                            uint32_t raw[TT][4];
#pragma unroll
                            for (int t = 0; t < TT; ++t) {
                                const int ts = t0 + t < nsteps_t ? t0 + t : t0;   // steps beyond T repeat the window's first and are never stored
                                const unsigned char* __restrict__ src = static_cast<const unsigned char*>(sk_kernarg_ptr(0, ts));
#pragma unroll
                                for (int j = 0; j < 4; ++j) raw[t][j] = src[idx[j]];
                            }
#pragma unroll
                            for (int t = 0; t < TT; ++t)
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const sk_u32x4 d = sk_expand_bits<ONE>(((ok_bits >> j) & 1u) ? raw[t][j] : 0u);
                                    if ((ok_bits >> (4 + j)) & 1u) *reinterpret_cast<sk_u32x4*>(wlds + t * tile_t + ((jb + j) * 64 + lane) * 16) = d;
                                }
                        } else {
#pragma unroll
                            for (int t = 0; t < TT; ++t) {
                                const int ts = t0 + t < nsteps_t ? t0 + t : t0;
                                const unsigned char* __restrict__ src = static_cast<const unsigned char*>(sk_kernarg_ptr(0, ts));
                                sk_u32x4 raw[4];
#pragma unroll
                                for (int j = 0; j < 4; ++j) raw[j] = *reinterpret_cast<const sk_u32x4*>(src + static_cast<int64_t>(idx[j]) * 16);
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    sk_u32x4 d;
#pragma unroll
                                    for (int k = 0; k < 4; ++k) d[k] = ((ok_bits >> j) & 1u) ? raw[j][k] : 0u;
                                    if ((ok_bits >> (4 + j)) & 1u) *reinterpret_cast<sk_u32x4*>(wlds + t * tile_t + ((jb + j) * 64 + lane) * 16) = d;
                                }
                            }
                        }
                    }
                }
                __builtin_amdgcn_wave_barrier();   // LDS serves a wave's accesses in order: the reads below see these writes
            };

            // ---- matrix loop over this wave's stages. Step = one pair of k-slots = one matrix instruction per (timestep,
            // 32-channel fragment); weight fragments stream from L2 two steps ahead through three register sets, across stages.
            if (have) {
                const int s_first = SK ? wk : 0;
                const int s_step = SK ? WK : 1;
                const int my_stages = s_first < g.nstages ? (g.nstages - s_first + s_step - 1) / s_step : 0;
                const int total = my_stages * nst;
                // Weight fragment of flat step `fs` of this wave (clamped to its last step).
                auto load_a = [&](int fs, sk_u32x4& a0, sk_u32x4& a1) __attribute__((always_inline)) {
                    fs = min(fs, total - 1);
                    const int si = fast_div(fs, g.d_nst);
                    const int st = fs - si * nst;
                    const int gg0 = (s_first + si * s_step) * g.G;
                    const int chunk = fast_div(gg0, g.d_gpc);
                    int pair;
                    if (g.tap_pairs) {
                        pair = chunk * g.npairs + st;
                    } else {
                        const int tap = fast_div(st, g.d_hg);
                        const int gp = st - tap * hg;
                        pair = chunk * g.npairs + ((tap * g.gpc + (gg0 - chunk * g.gpc) + 2 * gp) >> 1);
                    }
                    const int64_t o = static_cast<int64_t>(pair) * (kFragBytes / 2);
                    a0 = *reinterpret_cast<const sk_u32x4*>(wlane + w_off0 + o);
                    a1 = *reinterpret_cast<const sk_u32x4*>(wlane + w_off1 + o);
                };
                // Matrix work of step `st` of the stage in LDS.
                auto mma_step = [&](int st, const sk_u32x4& a0, const sk_u32x4& a1) __attribute__((always_inline)) {
                    const unsigned char* __restrict__ bq;
                    if (g.tap_pairs) {
                        const int tap0 = 2 * st, tap1 = min(2 * st + 1, g.taps - 1);   // an odd tap count leaves the last k-slot empty (zero weights)
                        const int kh0 = fast_div(tap0, g.d_KW), kh1 = fast_div(tap1, g.d_KW);
                        const int off0 = (kh0 * g.RC + (tap0 - kh0 * g.KW)) * 16;
                        const int off1 = (kh1 * g.RC + (tap1 - kh1 * g.KW)) * 16;
                        bq = wlds + lane_b + (half ? off1 : off0);
                    } else {
                        const int tap = fast_div(st, g.d_hg);
                        const int gp = st - tap * hg;
                        const int kh = fast_div(tap, g.d_KW);
                        bq = wlds + lane_b + (kh * g.RC + (tap - kh * g.KW)) * 16 + (2 * gp + half) * region16;
                    }
#pragma unroll
                    for (int t = 0; t < TT; ++t) {
                        const sk_u32x4 b = *reinterpret_cast<const sk_u32x4*>(bq + t * tile_t);
                        acc[t][0] = sk_mfma<F16>(a0, b, acc[t][0]);
                        acc[t][1] = sk_mfma<F16>(a1, b, acc[t][1]);
                    }
                };
                sk_u32x4 wa[3][2];
                if (total > 0) {
                    load_a(0, wa[0][0], wa[0][1]);
                    load_a(1, wa[1][0], wa[1][1]);
                }
                int st = 0;            // step inside the current stage
                int stage = s_first;
                for (int fs = 0; fs < total; fs += 3) {
                    load_a(fs + 2, wa[2][0], wa[2][1]);
                    if (st == 0) stage_in(stage);
                    mma_step(st, wa[0][0], wa[0][1]);
                    if (++st == nst) { st = 0; stage += s_step; }
                    if (fs + 1 < total) {
                        load_a(fs + 3, wa[0][0], wa[0][1]);
                        if (st == 0) stage_in(stage);
                        mma_step(st, wa[1][0], wa[1][1]);
                        if (++st == nst) { st = 0; stage += s_step; }
                    }
                    if (fs + 2 < total) {
                        load_a(fs + 4, wa[1][0], wa[1][1]);
                        if (st == 0) stage_in(stage);
                        mma_step(st, wa[2][0], wa[2][1]);
                        if (++st == nst) { st = 0; stage += s_step; }
                    }
                }
            }

            // ---- epilogue. Accumulator register 4 q + k of fragment f holds channel 32 f + 8 q + 4 half + k of the lane's
            // pixel: a "quad" (f, q) is the lane's half of channel group j8 = 8 oc_tile + 4 f + q. One quad at a time: its bias
            // and membrane (4 + 4 registers) live across its timesteps; a lane's addresses are 32-bit offsets from uniform bases.
            const float* __restrict__ v_src = t0 == 0 ? v_init : v_out;   // later windows continue from the stored membrane
            // The epilogue's loop-invariant loads (bias values of 8 quads) must not be hoisted above the matrix loop, where
            // they would hold registers: the pointer is made opaque here.
            const float* bias_e = bias;
            asm volatile("" : "+s"(bias_e));
            const int t_count = g.shared_x ? g.T : min(TT, g.T - t0);      // LIF steps of this window
            const uint32_t lane_nchw = static_cast<uint32_t>((n_c * g.Cout + 4 * half) * po + pxo);        // elements
            const uint32_t lane_c8 = static_cast<uint32_t>(((n_c * g.C8out) * po + pxo) * 8 + 4 * half);   // elements
            const uint32_t lane_bits = static_cast<uint32_t>((n_c * g.C8out) * po + pxo);                  // bytes

            // Bias, valid-channel mask and initial membrane of the quad of channel group j8.
            auto quad_begin = [&](int j8, float (&bv)[4], float (&v)[4], uint32_t& chm) __attribute__((always_inline)) {
                const int ch0 = j8 * 8 + 4 * half;
                chm = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const bool ch_ok = ch0 + k < g.Cout;
                    chm |= ch_ok ? (1u << k) : 0u;
                    bv[k] = ch_ok ? bias_e[ch0 + k] : 0.0f;
                    v[k] = 0.0f;
                }
                if (v_src != nullptr && !g.analog_out && px_ok) {
                    const float* __restrict__ vp = v_src + static_cast<int64_t>(j8) * 8 * po;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if ((chm >> k) & 1u) v[k] = vp[lane_nchw + static_cast<uint32_t>(k * po)];
                }
            };
            // One step of a quad at absolute timestep `ta`: x = sums + bias (+ residual), then the neuron (its spikes are the
            // returned nibble) or, without a neuron, x itself; dense output layouts are written here.
            auto quad_step = [&](int ta, int j8, const float (&x_in)[4], const float (&bv)[4], float (&v)[4], uint32_t chm) __attribute__((always_inline)) -> uint32_t {
                const bool grp_ok = j8 < g.C8out && px_ok;
                float x[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) x[k] = x_in[k] + bv[k];
                if (g.res_layout >= 0 && grp_ok) {
                    const unsigned char* __restrict__ res_t = static_cast<const unsigned char*>(sk_kernarg_ptr(kResTable, ta));
                    if (g.res_layout == SNNF_LAYOUT_BITS) {
                        const uint32_t byte = (res_t + static_cast<int64_t>(j8) * po)[lane_bits];
#pragma unroll
                        for (int k = 0; k < 4; ++k) x[k] += ((byte >> (4 * half + k)) & 1u) ? 1.0f : 0.0f;
                    } else if (g.res_layout == SNNF_LAYOUT_C8) {
                        const Pack<XT, 4> r4 = *reinterpret_cast<const Pack<XT, 4>*>(reinterpret_cast<const XT*>(res_t) + static_cast<int64_t>(j8) * po * 8 + lane_c8);
#pragma unroll
                        for (int k = 0; k < 4; ++k) x[k] += to_float(r4.v[k]);
                    } else {
                        const XT* __restrict__ rp = reinterpret_cast<const XT*>(res_t) + static_cast<int64_t>(j8) * 8 * po;
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            if ((chm >> k) & 1u) x[k] += to_float(rp[lane_nchw + static_cast<uint32_t>(k * po)]);
                    }
                }
                uint32_t nib = 0;
                if (!g.analog_out) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) nib |= lif_step(x[k], v[k], lif) ? (1u << k) : 0u;
                    nib &= chm;
                }
                if (grp_ok && g.out_layout != SNNF_LAYOUT_BITS) {
                    unsigned char* __restrict__ out_t = out + static_cast<int64_t>(ta) * g.out_step_stride;
                    Pack<XT, 4> o;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        o.v[k] = g.analog_out ? from_float<XT>(((chm >> k) & 1u) ? x[k] : 0.0f) : spike_value<XT>((nib >> k) & 1u);
                    if (g.out_layout == SNNF_LAYOUT_C8) {
                        *reinterpret_cast<Pack<XT, 4>*>(reinterpret_cast<XT*>(out_t) + static_cast<int64_t>(j8) * po * 8 + lane_c8) = o;
                    } else {
                        XT* __restrict__ op = reinterpret_cast<XT*>(out_t) + static_cast<int64_t>(j8) * 8 * po;
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            if ((chm >> k) & 1u) op[lane_nchw + static_cast<uint32_t>(k * po)] = o.v[k];
                    }
                }
                return nib;
            };
            // Bit-packed output of up to 8 consecutive steps [ta0, ta0 + cnt) of a quad: nibble i of `nibw` = step ta0 + i. The
            // other half of the wave holds the other nibble of every byte (lanes l and l + 32 own the same pixel); even
            // steps are stored by the lower half, odd steps by the upper half.
            auto quad_store_bits = [&](int ta0, int cnt, int j8, uint32_t nibw) __attribute__((always_inline)) {
                const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(nibw), 32));
                const uint32_t lo = half ? other : nibw;
                const uint32_t hi = half ? nibw : other;
                if (j8 < g.C8out && px_ok) {
                    unsigned char* __restrict__ ob = out + static_cast<int64_t>(j8) * po;
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        const int i = 2 * m + half;
                        if (i < cnt) {
                            const uint32_t byte = ((lo >> (4 * i)) & 15u) | (((hi >> (4 * i)) & 15u) << 4);
                            ob[static_cast<uint32_t>(ta0 + i) * static_cast<uint32_t>(g.out_step_stride) + lane_bits] = static_cast<unsigned char>(byte);
                        }
                    }
                }
            };
            auto quad_end = [&](int j8, const float (&v)[4], uint32_t chm) __attribute__((always_inline)) {
                if (v_out != nullptr && !g.analog_out && px_ok) {
                    float* __restrict__ vp = v_out + static_cast<int64_t>(j8) * 8 * po;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if ((chm >> k) & 1u) vp[lane_nchw + static_cast<uint32_t>(k * po)] = v[k];
                }
            };

            if constexpr (!SK) {
                // A runtime loop over the wave's 8 quads keeps the code small; a quad's sums are copied out of the accumulators
                // by a switch (constant register indices), so the accumulators stay in registers.
                for (int fq = 0; fq < 8; ++fq) {
                    const int j8 = oc_tile * 8 + fq;
                    float xq[TT][4];
#define SNNF_SPK_COPY_QUAD(F, Q)                                          \
    _Pragma("unroll") for (int tw = 0; tw < TT; ++tw)                     \
        _Pragma("unroll") for (int k = 0; k < 4; ++k) xq[tw][k] = acc[tw][F][4 * (Q) + k]
                    switch (fq) {
                        case 0: SNNF_SPK_COPY_QUAD(0, 0); break;
                        case 1: SNNF_SPK_COPY_QUAD(0, 1); break;
                        case 2: SNNF_SPK_COPY_QUAD(0, 2); break;
                        case 3: SNNF_SPK_COPY_QUAD(0, 3); break;
                        case 4: SNNF_SPK_COPY_QUAD(1, 0); break;
                        case 5: SNNF_SPK_COPY_QUAD(1, 1); break;
                        case 6: SNNF_SPK_COPY_QUAD(1, 2); break;
                        default: SNNF_SPK_COPY_QUAD(1, 3); break;
                    }
#undef SNNF_SPK_COPY_QUAD
                    float bv[4], v[4];
                    uint32_t chm;
                    quad_begin(j8, bv, v, chm);
                    if constexpr (TT == 1) {
                        // One convolution result, t_count LIF steps on it (one step, or one frame shared by all T timesteps).
                        for (int ta0 = 0; ta0 < t_count; ta0 += 8) {
                            const int cnt = min(8, t_count - ta0);
                            uint32_t nibw = 0;
                            for (int i = 0; i < cnt; ++i) nibw |= quad_step(t0 + ta0 + i, j8, xq[0], bv, v, chm) << (4 * i);
                            if (g.out_layout == SNNF_LAYOUT_BITS) quad_store_bits(t0 + ta0, cnt, j8, nibw);
                        }
                    } else {
                        uint32_t nibw = 0;
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw)
                            if (tw < t_count) nibw |= quad_step(t0 + tw, j8, xq[tw], bv, v, chm) << (4 * tw);
                        if (g.out_layout == SNNF_LAYOUT_BITS) quad_store_bits(t0, t_count, j8, nibw);
                    }
                    quad_end(j8, v, chm);
                }
            } else {
                // Split K: every wave parks one timestep's 32 partial sums per lane in LDS (the staging regions are dead by
                // then); the owner of a quad adds the WK partial sums in a fixed order and runs that step's LIF right away, so
                // only the owned quads' membranes stay in registers between rounds.
                float* __restrict__ part = reinterpret_cast<float*>(lds);      // [wave][quad 0..7][lane][4]
                const int nq = 8 >> g.wk_log2;                                 // quads this wave owns: quad0 .. quad0 + nq - 1
                const int quad0 = wk * nq;
                float bv[4][4], v[4][4];
                uint32_t chm[4], nibw[4];
#pragma unroll
                for (int qi = 0; qi < 4; ++qi) {
                    nibw[qi] = 0;
                    if (qi < nq) quad_begin(oc_tile * 8 + quad0 + qi, bv[qi], v[qi], chm[qi]);
                }
#pragma unroll
                for (int tw = 0; tw < TT; ++tw) {
                    if (tw < (TT == 1 ? 1 : t_count)) {   // uniform over the workgroup
                        __syncthreads();
#pragma unroll
                        for (int f = 0; f < 2; ++f)
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const sk_f32x4 four = {acc[tw][f][4 * q], acc[tw][f][4 * q + 1], acc[tw][f][4 * q + 2], acc[tw][f][4 * q + 3]};
                                *reinterpret_cast<sk_f32x4*>(part + ((wave * 8 + f * 4 + q) * 64 + lane) * 4) = four;
                            }
                        __syncthreads();
#pragma unroll
                        for (int qi = 0; qi < 4; ++qi) {
                            if (qi < nq) {
                                const int j8 = oc_tile * 8 + quad0 + qi;
                                sk_f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
                                for (int k = 0; k < WK; ++k)
                                    sum += *reinterpret_cast<const sk_f32x4*>(part + (((tile_in_block * WK + k) * 8 + quad0 + qi) * 64 + lane) * 4);
                                const float x_in[4] = {sum[0], sum[1], sum[2], sum[3]};
                                if constexpr (TT == 1) {
                                    for (int ta0 = 0; ta0 < t_count; ta0 += 8) {
                                        const int cnt = min(8, t_count - ta0);
                                        uint32_t w8 = 0;
                                        for (int i = 0; i < cnt; ++i) w8 |= quad_step(t0 + ta0 + i, j8, x_in, bv[qi], v[qi], chm[qi]) << (4 * i);
                                        if (g.out_layout == SNNF_LAYOUT_BITS) quad_store_bits(t0 + ta0, cnt, j8, w8);
                                    }
                                } else {
                                    nibw[qi] |= quad_step(t0 + tw, j8, x_in, bv[qi], v[qi], chm[qi]) << (4 * tw);
                                }
                            }
                        }
                    }
                }
#pragma unroll
                for (int qi = 0; qi < 4; ++qi) {
                    if (qi < nq) {
                        const int j8 = oc_tile * 8 + quad0 + qi;
                        if (TT > 1 && g.out_layout == SNNF_LAYOUT_BITS) quad_store_bits(t0, t_count, j8, nibw[qi]);
                        quad_end(j8, v[qi], chm[qi]);
                    }
                }
            }
            if constexpr (SK) __syncthreads();   // the partial sums are read before the next window's staging overwrites them
        }
    }
}

template <typename XT, int TT, int IN>
int launch_conv_spk_variant(const SpkLaunch& L) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif_blocked"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kSpkWaves * 64, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.g, L.wpacked, L.bias, L.v_init,
                                                                        static_cast<unsigned char*>(L.out), L.v_out, L.lif);
        return check_launch("snnf_conv_lif_blocked");
    };
    return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, TT, IN, true>) : run(conv_spk_kernel<XT, TT, IN, false>);
}

template <typename XT>
int launch_conv_spk_tt(const SpkLaunch& L, int tt) {
    if (L.g.in_layout == SNNF_LAYOUT_BITS) {
        if (tt == 4) return launch_conv_spk_variant<XT, 4, SNNF_LAYOUT_BITS>(L);
        if (tt == 2) return launch_conv_spk_variant<XT, 2, SNNF_LAYOUT_BITS>(L);
        return launch_conv_spk_variant<XT, 1, SNNF_LAYOUT_BITS>(L);
    }
    if (tt == 4) return launch_conv_spk_variant<XT, 4, SNNF_LAYOUT_C8>(L);
    if (tt == 2) return launch_conv_spk_variant<XT, 2, SNNF_LAYOUT_C8>(L);
    return launch_conv_spk_variant<XT, 1, SNNF_LAYOUT_C8>(L);
}

int launch_conv_spk_bf16(const SpkLaunch& L, int tt);
int launch_conv_spk_f16(const SpkLaunch& L, int tt);

}  // namespace snnf
