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
//     sums through LDS in a fixed order, one timestep per round;
//   * neighbours of a convolution that fit its tile join its launch: the 1x1 projection shortcut of a residual block as
//     further K steps on a second input (SC), the 2x2 average pool of the spikes as a reduce-scatter between the four
//     lanes of a window (POOL), and a network's dense input frame of at most 8 channels read as it is (IN = NCHW).
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
constexpr size_t kSpkPartialBytes = kSpkWaves * 16 * 64 * 16;  // split-K: every wave parks 4 quads x up to 4 timesteps of partial sums per round
constexpr int kSpkMaxSteps = 60;                  // matrix steps per stage, at most (the step table holds 4 more)
constexpr size_t kSpkTableBytes = (kSpkMaxSteps + 4) * 16;      // the workgroup's step table at the start of LDS
constexpr int kSpkDescs = 64 * kSpkSlots;                       // staging items of one timestep, at most
constexpr size_t kSpkDescBytes = kSpkDescs * 8;                 // the workgroup's staging descriptors behind the step table
constexpr size_t kSpkPosBytes = 32 * 4;            // where each of the 32 pixels of a tile sits inside the patch
constexpr size_t kSpkHeaderBytes = kSpkTableBytes + kSpkDescBytes + kSpkPosBytes;   // what precedes the waves' staging regions in LDS

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
    int kw_mul;                  // tap / KW == (tap * kw_mul) >> 16 for every tap of the kernel (branch-free on the scalar unit)
    int gpc_log2;                // log2(gpc)
    int hg_log2;                 // log2 of the k-slot pairs per tap and stage (G / 2; 0 with tap pairs)
    int pair_tap_stride;         // packed pairs between consecutive taps of one group pair (gpc / 2; 1 with tap pairs)
    int wk_log2;                 // split-K: waves per tile
    int n_items, iters;          // (patch, 64-channel tile) pairs; loop trips per wave
    int in_layout, res_layout, out_layout;   // snnf_layout codes; res_layout < 0: no residual
    int analog_out;              // no neuron: the sums themselves are written (C8 or NCHW)
    int pool2;                   // the POOL variants: the spikes leave as their 2x2 averages (quarters, C8, half the plane)
    int64_t out_step_stride;     // bytes between timesteps of `out`
    int lds_wave_bytes;          // private staging region of a wave (a multiple of 16)
    int64_t frag_stride;         // 16-bit elements between consecutive 32-row fragments of the packed weight
    // A second, pointwise operand pair that shares the accumulators (the projection shortcut of a residual block: its sums
    // are further K steps of the same output tile). Its input has sc_C8 channel groups on an sc_H x sc_W plane and is
    // sampled at (sc_sh * ih, sc_sw * iw) for the pixel (ih, iw) of the main input; its stages follow the main ones.
    int sc_stages;               // 0: none
    int sc_C8, sc_H, sc_W, sc_sh, sc_sw;
    int sc_gpc_log2, sc_npairs;  // channel groups (log2) and k-slot pairs per packed chunk of the second weight
    int64_t sc_frag_stride;
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
    const uint16_t* wpacked2;   // packed weight and bias of the shortcut (sc_stages > 0), else null
    const float* bias2;
    int grid;
    size_t lds_bytes;
    hipStream_t stream;
    bool fast_epilogue;   // the straight-line epilogue applies: bit-packed output, no or a bit-packed residual, the usual neuron
                          // (tau 2, hard reset to 0), zero initial membrane, one window, whole channel groups
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
// fast_div without a branch: the multiply-high runs for a divisor of 1 as well (its multiplier is 0, the quotient then
// comes from the mask). The staging decode divides three times per item; a uniform branch around each of them costs more
// than the multiply and keeps the compiler from overlapping the items.
__device__ __forceinline__ int sk_div(int n, const FastDiv& f) {
    const uint32_t keep = f.d == 1u ? 0xffffffffu : 0u;
    return static_cast<int>((__umulhi(static_cast<uint32_t>(n), f.mul) >> f.shift) | (static_cast<uint32_t>(n) & keep));
}

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

template <typename XT, int TT, int IN, bool SK, bool FAST, bool SC = false, bool POOL = false>
__global__ __launch_bounds__(kSpkWaves * 64, 1) __attribute__((amdgpu_waves_per_eu(TT == 1 ? 4 : 2, TT == 1 ? 4 : 2))) void conv_spk_kernel(
    const StepPtrs xs, const StepPtrs residuals, const SpkGeom g, const uint16_t* __restrict__ wpacked,
    const float* __restrict__ bias, const float* __restrict__ v_init, unsigned char* __restrict__ out,
    float* __restrict__ v_out, const LifParams lif, const uint16_t* __restrict__ wpacked2, const float* __restrict__ bias2) {
    extern __shared__ __align__(16) unsigned char lds[];
    // ---- every cache line of the kernel arguments is touched once, in one round trip: the compiler loads the arguments
    // where they are used, all over the prologue, and each of those loads then hits the scalar cache instead of waiting
    // for memory in turn.
    {
        auto ka = __builtin_amdgcn_kernarg_segment_ptr();
        // The explicit arguments are two step tables, the geometry, five pointers and the neuron: the last dword that is
        // touched must lie inside them (what follows is the hidden-argument area, which the compiler may leave out).
        constexpr size_t kExplicitArgBytes = 2 * sizeof(StepPtrs) + sizeof(SpkGeom) + 7 * sizeof(void*) + sizeof(LifParams);
        static_assert(0x2c0 + 4 <= kExplicitArgBytes, "argument prefetch reads past the explicit kernel arguments");
        static_assert(kExplicitArgBytes <= 0x300, "argument prefetch does not cover the last cache line of the arguments");
        uint32_t d0, d1, d2, d3, d4, d5, d6, d7, d8, d9, d10;
        asm volatile(
            "s_load_dword %0, %11, 0x40\n\ts_load_dword %1, %11, 0x80\n\ts_load_dword %2, %11, 0xc0\n\ts_load_dword %3, %11, 0x100\n\t"
            "s_load_dword %4, %11, 0x140\n\ts_load_dword %5, %11, 0x180\n\ts_load_dword %6, %11, 0x1c0\n\ts_load_dword %7, %11, 0x200\n\t"
            "s_load_dword %8, %11, 0x240\n\ts_load_dword %9, %11, 0x280\n\ts_load_dword %10, %11, 0x2c0\n\ts_waitcnt lgkmcnt(0)"
            : "=&s"(d0), "=&s"(d1), "=&s"(d2), "=&s"(d3), "=&s"(d4), "=&s"(d5), "=&s"(d6), "=&s"(d7), "=&s"(d8), "=&s"(d9), "=&s"(d10)
            : "s"(ka));
    }
    __builtin_amdgcn_sched_barrier(0);

    static_assert(!SC || (IN == SNNF_LAYOUT_BITS && TT == 4), "the shortcut variants take bit-packed inputs, four timesteps at a time");
    static_assert(!POOL || (FAST && (TT == 4 || TT == 1)), "the pooled output belongs to the straight-line epilogue of four steps");
    static_assert(IN != SNNF_LAYOUT_NCHW || TT == 1, "a dense input is one frame for all timesteps");
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    constexpr uint32_t ONE = F16 ? 0x3c00u : 0x3f80u;
    constexpr int kResTable = static_cast<int>(sizeof(StepPtrs));
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int l32 = lane & 31;
    unsigned char* const wlds = lds + kSpkHeaderBytes + wave * g.lds_wave_bytes;
    const int region16 = g.region * 16;        // bytes of one channel group of the halo
    const int tile_t = g.G * region16 + 16;    // bytes of one timestep's stage: its items and one dummy item that absorbs the writes of idle staging slots

    const int WK = SK ? (1 << g.wk_log2) : 1;
    const int wk = SK ? (wave & (WK - 1)) : 0;
    const int tile_in_block = SK ? (wave >> g.wk_log2) : wave;
    const int tiles_per_block = SK ? (kSpkWaves >> g.wk_log2) : kSpkWaves;
    const int po = g.Ho * g.Wo;
    const int nsteps_t = g.shared_x ? 1 : g.T;          // timesteps with a convolution of their own
    const int hg = g.tap_pairs ? 1 : (g.G >> 1);        // k-slot pairs per tap and stage
    const int nst = g.tap_pairs ? g.npairs : g.taps * hg;   // matrix steps per stage
    const bool common_lif = lif.charge_mode == CHARGE_SCALE && !lif.soft_reset;
    const bool half_tau = lif.inv_tau == 0.5f;

    // ---- step table of the workgroup: for step i of a stage, the byte offset of its weight fragments from the stage's
    // first pair and the LDS offset of its activations (tap and channel group of the half's k-slot), once for the lower and
    // once for the upper half of a wave: a lane reads the 8 bytes of its half. The matrix loop then needs no index
    // arithmetic. Steps beyond the last repeat it (prefetch only).
    {
        sk_u32x4* __restrict__ table = reinterpret_cast<sk_u32x4*>(lds);
        if (tid < nst + 4) {
            const int i = min(tid, nst - 1);
            sk_u32x4 e;
            if (g.tap_pairs) {
                const int tap0 = 2 * i, tap1 = min(2 * i + 1, g.taps - 1);   // an odd tap count leaves the last k-slot empty (zero weights)
                const int kh0 = tap0 / g.KW, kh1 = tap1 / g.KW;
                e[0] = static_cast<uint32_t>(i * kFragBytes);
                e[1] = static_cast<uint32_t>((kh0 * g.RC + (tap0 - kh0 * g.KW)) * 16);
                e[3] = static_cast<uint32_t>((kh1 * g.RC + (tap1 - kh1 * g.KW)) * 16);
            } else {
                const int tap = i >> g.hg_log2;
                const int gp = i & (hg - 1);
                const int kh = tap / g.KW;
                const int tapoff = (kh * g.RC + (tap - kh * g.KW)) * 16;
                e[0] = static_cast<uint32_t>((tap * g.pair_tap_stride + gp) * kFragBytes);
                e[1] = static_cast<uint32_t>(tapoff + (2 * gp) * region16);
                e[3] = static_cast<uint32_t>(tapoff + (2 * gp + 1) * region16);
            }
            e[2] = e[0];
            table[tid] = e;
        }
        if constexpr (SC) {
            // The shortcut's stages: one tap, the centre of the main kernel (the lane's own pixel), on the same halo; entries
            // behind the main table's.
            const int i2 = tid - (nst + 4);
            if (i2 >= 0 && i2 < hg + 4) {
                const int gp = min(i2, hg - 1);
                const int tapoff = (g.ph * g.RC + g.pw) * 16;
                sk_u32x4 e;
                e[0] = static_cast<uint32_t>(gp * kFragBytes);
                e[1] = static_cast<uint32_t>(tapoff + (2 * gp) * region16);
                e[2] = e[0];
                e[3] = static_cast<uint32_t>(tapoff + (2 * gp + 1) * region16);
                table[tid] = e;
            }
        }
        // ---- staging descriptors of the workgroup: item e of a timestep's stage = (channel group gq, image ii, halo row r, halo
        // column c); its element offset from the stage's first item and the four coordinates, packed. Built once; the staging
        // of every stage of every tile reads them back instead of dividing (three divisions per item otherwise). Items beyond
        // the stage carry channel group 255, which no stage has.
        Pack<uint32_t, 2>* __restrict__ desc_w = reinterpret_cast<Pack<uint32_t, 2>*>(lds + kSpkTableBytes);
        for (int e = tid; e < kSpkDescs; e += kSpkWaves * 64) {
            Pack<uint32_t, 2> d;
            d.v[0] = 0u;
            d.v[1] = 0xff000000u;
            if (e < g.IT) {
                const int gq = sk_div(e, g.d_region);
                const int rem = e - gq * g.region;
                const int ii = sk_div(rem, g.d_rrrc);
                const int rem2 = rem - ii * (g.RR * g.RC);
                const int r = sk_div(rem2, g.d_RC);
                const int c = rem2 - r * g.RC;
                if constexpr (IN == SNNF_LAYOUT_NCHW) d.v[0] = static_cast<uint32_t>(((ii * g.Cin + gq * 8) * g.H + r) * g.W + c);   // elements of a dense frame
                else d.v[0] = static_cast<uint32_t>(((ii * g.C8in + gq) * g.H + r) * g.W + c);
                d.v[1] = static_cast<uint32_t>(r) | (static_cast<uint32_t>(c) << 8) | (static_cast<uint32_t>(ii) << 16) | (static_cast<uint32_t>(gq) << 24);
            }
            desc_w[e] = d;
        }
        // ---- where pixel p of a tile sits inside the patch: image, row and column, packed. Every item reads its lane's entry
        // back: kept in registers these values would live (or be spilled) across the matrix loop of every variant.
        if (tid < 32) {
            const int ppx = g.PR * g.PC;
            const int pi = sk_div(tid, g.d_ppx);
            const int prem = tid - pi * ppx;
            const int prow = sk_div(prem, g.d_PC);
            const int pcol = prem - prow * g.PC;
            reinterpret_cast<uint32_t*>(lds + kSpkTableBytes + kSpkDescBytes)[tid] =
                static_cast<uint32_t>(pi) | (static_cast<uint32_t>(prow) << 8) | (static_cast<uint32_t>(pcol) << 16);
        }
        __syncthreads();
    }
    const Pack<uint32_t, 2>* __restrict__ desc = reinterpret_cast<const Pack<uint32_t, 2>*>(lds + kSpkTableBytes);
    const Pack<uint32_t, 2>* __restrict__ table = reinterpret_cast<const Pack<uint32_t, 2>*>(lds + 8 * half);   // entry i of this half: table[2 * i]

    // Workgroups are handed to the eight XCDs in turn (workgroup b runs on XCD b % 8) and every XCD has an L2 of its own.
    // Items are ordered output-channel tile first, so the workgroups of one XCD take a contiguous range of them: an XCD then
    // reads the weights of few output-channel tiles (one, for a 512-channel layer) instead of the whole tensor.
    const int nb = static_cast<int>(gridDim.x);
    const int xcd = static_cast<int>(blockIdx.x) & 7;
    const int block_l = xcd * (nb >> 3) + min(xcd, nb & 7) + (static_cast<int>(blockIdx.x) >> 3);
    for (int it = 0; it < g.iters; ++it) {
        // Consecutive items go to different workgroups, so that a layer with fewer items than wave slots still uses every compute unit.
        const int item = (it * tiles_per_block + tile_in_block) * nb + block_l;
        const bool have = item < g.n_items;
        const int item_c = have ? item : 0;
        const int oc_tile = sk_div(item_c, g.d_n_patches);
        const int patch = item_c - oc_tile * g.n_patches;
        const int imgg = sk_div(patch, g.d_patches_img);
        const int prem_i = patch - imgg * g.patches_img;
        const int py = sk_div(prem_i, g.d_patches_x);
        const int n0 = imgg * g.PI;
        const int oh0 = py * g.PR;
        const int ow0 = (prem_i - py * g.patches_x) * g.PC;
        const int ih_lo = oh0 * g.sh - g.ph;
        const int iw_lo = ow0 * g.sw - g.pw;

        // ---- this lane's output pixel inside the patch, and where its top-left input sits in the staged halo.
        const uint32_t lane_pos = reinterpret_cast<const uint32_t*>(lds + kSpkTableBytes + kSpkDescBytes)[l32];
        const int pi = static_cast<int>(lane_pos & 255u);
        const int prow = static_cast<int>((lane_pos >> 8) & 255u);
        const int pcol = static_cast<int>(lane_pos >> 16);
        const bool lane_in_patch = pi < g.PI;
        const uint32_t lane_b = lane_in_patch ? static_cast<uint32_t>(((pi * g.RR + prow * g.sh) * g.RC + pcol * g.sw) * 16) : 0u;

        const int ocf0 = oc_tile * 2;
        // With K split over two waves the second one computes the tile's two 32-channel fragments in swapped places: each wave
        // then finishes the fragment in its accumulators' first half (fragment wk) and hands over the second half.
        const int swap_f = (SK && WK == 2) ? wk : 0;
        const int64_t w_frag0 = min(ocf0 + swap_f, g.nocf - 1);
        const int64_t w_frag1 = min(ocf0 + 1 - swap_f, g.nocf - 1);

        // ---- this lane's output pixel.
        const int n = n0 + pi;
        const int oh = oh0 + prow;
        const int ow = ow0 + pcol;
        const bool px_ok = have && lane_in_patch && n < g.N && oh < g.Ho && ow < g.Wo;
        const int pxo = px_ok ? oh * g.Wo + ow : 0;
        const int n_c = px_ok ? n : 0;

        for (int t0 = 0; t0 < nsteps_t; t0 += TT) {
            // The accumulators start from the bias: register 4 q + k of fragment f is channel 64 oc_tile + 32 f + 8 q + 4 half + k.
            // With K split over waves only the first one adds it. The bias is requested here and copied into the accumulators
            // after the first stage's activations have been requested, so that both round trips to memory overlap.
            sk_f32x16 acc[TT][2];
            sk_f32x4 bias4[2][4];
            {
                const int nbias = g.nocf * 32;               // bias values behind the packed weight (zero beyond Cout)
#pragma unroll
                for (int f = 0; f < 2; ++f)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int ch0 = oc_tile * 64 + f * 32 + q * 8 + 4 * half;
                        bias4[f][q] = sk_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                        if (ch0 < nbias && (!SK || wk == 0)) bias4[f][q] = *reinterpret_cast<const sk_f32x4*>(bias + ch0);
                    }
                if constexpr (SC) {
                    sk_f32x4 more[2][4];
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int ch0 = oc_tile * 64 + f * 32 + q * 8 + 4 * half;
                            more[f][q] = sk_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                            if (ch0 < nbias && (!SK || wk == 0)) more[f][q] = *reinterpret_cast<const sk_f32x4*>(bias2 + ch0);
                        }
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int q = 0; q < 4; ++q) bias4[f][q] += more[f][q];
                }
            }

            // One LDS stage: G channel groups of the patch's halo for TT timesteps, from global memory into this wave's region.
            // Item e = slot * 64 + lane of a timestep = (group, image, row, column) of the halo; its LDS address is 16 e. Items
            // are decoded on the fly (nothing about them is kept in registers across the matrix loop) and move in batches of 4
            // slots x TT timesteps: all loads of a batch are in flight together.
            // PRE (bit-packed inputs, lean epilogue): the first batch of the NEXT stage is requested before the matrix steps of the
            // current one and sits in registers meanwhile, so that its latency hides behind them.
            constexpr bool PRE = FAST && IN == SNNF_LAYOUT_BITS;
            uint32_t pre_raw[TT][4];
            uint32_t pre_ok = 0;
            // Decodes the 4 items of batch jb of stage s from the workgroup's descriptors: their global index (0 when they are
            // padding) and a flag nibble (bit j: real data).
            // A stage at or beyond g.nstages (SC only) is one of the shortcut's: same halo items, taken from the second input at
            // the sampled positions.
            auto batch_decode = [&](int s, int jb, int lane_s, int (&idx)[4]) __attribute__((always_inline)) -> uint32_t {
                const bool second = SC && s >= g.nstages;
                const int gg0 = (second ? s - g.nstages : s) * g.G;
                const int c8 = second ? g.sc_C8 : g.C8in;
                const int base_u = second ? ((n0 * g.sc_C8 + gg0) * g.sc_H + ih_lo * g.sc_sh) * g.sc_W + iw_lo * g.sc_sw
                                   : IN == SNNF_LAYOUT_NCHW ? ((n0 * g.Cin + gg0 * 8) * g.H + ih_lo) * g.W + iw_lo
                                          : ((n0 * g.C8in + gg0) * g.H + ih_lo) * g.W + iw_lo;   // may be negative; only added to in-image items
                uint32_t ok_bits = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const Pack<uint32_t, 2> d = desc[(jb + j) * 64 + lane_s];
                    const int r = static_cast<int>(d.v[1] & 255u), c = static_cast<int>((d.v[1] >> 8) & 255u);
                    const int ii = static_cast<int>((d.v[1] >> 16) & 255u), gq = static_cast<int>(d.v[1] >> 24);
                    const bool ok = n0 + ii < g.N && gg0 + gq < c8 && static_cast<unsigned>(ih_lo + r) < static_cast<unsigned>(g.H) &&
                                    static_cast<unsigned>(iw_lo + c) < static_cast<unsigned>(g.W);
                    int off = static_cast<int>(d.v[0]);
                    if constexpr (SC) {
                        if (second) off = ((ii * g.sc_C8 + gq) * g.sc_H + r * g.sc_sh) * g.sc_W + c * g.sc_sw;
                    }
                    idx[j] = ok ? base_u + off : 0;
                    ok_bits |= ok ? (1u << j) : 0u;
                }
                return ok_bits;
            };
            auto batch_load_bits = [&](int s, const int (&idx)[4], uint32_t (&raw)[TT][4]) __attribute__((always_inline)) {
                const int ptr_table = SC && s >= g.nstages ? kResTable : 0;
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const int ts = t0 + t < nsteps_t ? t0 + t : t0;   // steps beyond T repeat the window's first and are never stored
                    const unsigned char* __restrict__ src = static_cast<const unsigned char*>(sk_kernarg_ptr(ptr_table, ts));
#pragma unroll
                    for (int j = 0; j < 4; ++j) raw[t][j] = src[idx[j]];
                }
            };
            auto batch_put_bits = [&](int jb, int lane_s, uint32_t ok_bits, const uint32_t (&raw)[TT][4]) __attribute__((always_inline)) {
#pragma unroll
                for (int t = 0; t < TT; ++t)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const sk_u32x4 d = sk_expand_bits<ONE>(((ok_bits >> j) & 1u) ? raw[t][j] : 0u);
                        // every slot writes: an item beyond the stage goes to the timestep's dummy item
                        *reinterpret_cast<sk_u32x4*>(wlds + t * tile_t + min((jb + j) * 64 + lane_s, g.IT) * 16) = d;
                    }
            };
            // Requests the first batch of stage s (PRE only).
            auto stage_req = [&](int s) __attribute__((always_inline)) {
                int lane_s = lane;
                asm volatile("" : "+v"(lane_s));
                int idx[4];
                pre_ok = batch_decode(s, 0, lane_s, idx);
                batch_load_bits(s, idx, pre_raw);
            };
            // One LDS stage: G channel groups of the patch's halo for TT timesteps, from global memory into this wave's region.
            // Item e = slot * 64 + lane of a timestep = (group, image, row, column) of the halo; its LDS address is 16 e. Items
            // are decoded on the fly (nothing about them is kept in registers across the matrix loop) and move in batches of 4
            // slots x TT timesteps: all loads of a batch are in flight together.
            auto stage_in = [&](int s) __attribute__((always_inline)) {
                __builtin_amdgcn_wave_barrier();   // the matrix steps of the previous stage have read their operands
                int lane_s = lane;                 // opaque: the decode below stays here instead of being hoisted out of every loop
                asm volatile("" : "+v"(lane_s));   // (its results would sit in registers, or in scratch memory, across the matrix loop)
#pragma unroll
                for (int jb = 0; jb < kSpkSlots; jb += 4) {
                    if (jb < g.JT) {
                        if constexpr (PRE) {
                            if (jb == 0) {
                                batch_put_bits(0, lane_s, pre_ok, pre_raw);
                                continue;
                            }
                        }
                        int idx[4];
                        const uint32_t ok_bits = batch_decode(s, jb, lane_s, idx);
                        if constexpr (IN == SNNF_LAYOUT_BITS) {
                            uint32_t raw[TT][4];
                            batch_load_bits(s, idx, raw);
                            batch_put_bits(jb, lane_s, ok_bits, raw);
                        } else if constexpr (IN == SNNF_LAYOUT_NCHW) {
                            // A dense frame of at most 8 channels (the network's input): one 16-bit load per channel and item.
                            const int plane = g.H * g.W;
#pragma unroll
                            for (int t = 0; t < TT; ++t) {
                                const int ts = t0 + t < nsteps_t ? t0 + t : t0;
                                const uint16_t* __restrict__ src = static_cast<const uint16_t*>(sk_kernarg_ptr(0, ts));
                                uint32_t h[4][8];
#pragma unroll
                                for (int k = 0; k < 8; ++k) {
                                    if (k < g.Cin) {
#pragma unroll
                                        for (int j = 0; j < 4; ++j) h[j][k] = src[idx[j] + k * plane];
                                    } else {
#pragma unroll
                                        for (int j = 0; j < 4; ++j) h[j][k] = 0u;
                                    }
                                }
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    sk_u32x4 d;
#pragma unroll
                                    for (int k = 0; k < 4; ++k) d[k] = ((ok_bits >> j) & 1u) ? (h[j][2 * k] | (h[j][2 * k + 1] << 16)) : 0u;
                                    *reinterpret_cast<sk_u32x4*>(wlds + t * tile_t + min((jb + j) * 64 + lane_s, g.IT) * 16) = d;
                                }
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
                                    *reinterpret_cast<sk_u32x4*>(wlds + t * tile_t + min((jb + j) * 64 + lane_s, g.IT) * 16) = d;
                                }
                            }
                        }
                    }
                }
                __builtin_amdgcn_wave_barrier();   // LDS serves a wave's accesses in order: the reads below see these writes
            };

            // ---- matrix loop over this wave's stages. Step = one pair of k-slots = one matrix instruction per (timestep,
            // 32-channel fragment). Per stage: the first weight fragments are requested from L2, the stage is brought into LDS,
            // then the steps run four at a time without a branch: weight fragments three steps ahead through four register
            // sets, activation fragments one step ahead through two.
            const int s_first = SK ? wk : 0;
            const int s_step = SK ? WK : 1;
            const int nstages_all = SC ? g.nstages + g.sc_stages : g.nstages;
            if constexpr (PRE) {
                if (have && s_first < nstages_all) stage_req(s_first);
            }
            // The epilogue's view of the tile's channel block, opaque from here on: the scalar arithmetic that depends on it
            // (per-quad base addresses and store predicates, several hundred scalar instructions that the compiler computes
            // ahead of time) then runs after the tile's first loads have been requested, under their latency, instead of in
            // front of them.
            int oc_e = oc_tile;
            asm volatile("" : "+s"(oc_e));
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int t = 0; t < TT; ++t)
#pragma unroll
                        for (int k = 0; k < 4; ++k) acc[t][f][4 * q + k] = bias4[f][q][k];
            if constexpr (!SK) {
                // The two waves of a SIMD unit (waves w and w + 4 of the workgroup) run out of phase: the first has the matrix
                // cores to itself and then runs its epilogue, on the vector unit, under the second one's matrix instructions.
                if (wave < 4) __builtin_amdgcn_s_setprio(2);
                else __builtin_amdgcn_s_setprio(1);
            }
            if (have) {
                const uint32_t lane16 = static_cast<uint32_t>(lane) * 16u;
                const unsigned char* __restrict__ bl = wlds + lane_b;
                for (int stage = s_first; stage < nstages_all; stage += s_step) {
                    const bool second = SC && stage >= g.nstages;     // a stage of the shortcut
                    const int gg0 = (second ? stage - g.nstages : stage) * g.G;
                    const int gpc_l2 = second ? g.sc_gpc_log2 : g.gpc_log2;
                    const int chunk = gg0 >> gpc_l2;
                    const int pbase = chunk * (second ? g.sc_npairs : g.npairs) + ((gg0 - (chunk << gpc_l2)) >> 1);   // pair of (tap 0, the stage's first two groups)
                    const uint16_t* __restrict__ wp = second ? wpacked2 : wpacked;
                    const int64_t fs = second ? g.sc_frag_stride : g.frag_stride;
                    const unsigned char* __restrict__ pa0 = reinterpret_cast<const unsigned char*>(wp + w_frag0 * fs + static_cast<int64_t>(pbase) * (kFragBytes / 2));
                    const unsigned char* __restrict__ pa1 = reinterpret_cast<const unsigned char*>(wp + w_frag1 * fs + static_cast<int64_t>(pbase) * (kFragBytes / 2));
                    const Pack<uint32_t, 2>* __restrict__ tb = second ? table + 2 * (nst + 4) : table;
                    const int nst_s = second ? hg : nst;
                    sk_u32x4 wa[4][2];
                    sk_u32x4 wb[2][TT];
                    uint32_t bo[4];
                    // Requests the weight fragments of the step described by table entry `e` and notes where its activations are.
                    auto req_a = [&](int slot, const Pack<uint32_t, 2>& e) __attribute__((always_inline)) {
                        const uint32_t voff = lane16 + e.v[0];
                        wa[slot][0] = *reinterpret_cast<const sk_u32x4*>(pa0 + voff);
                        wa[slot][1] = *reinterpret_cast<const sk_u32x4*>(pa1 + voff);
                        bo[slot] = e.v[1];
                    };
                    auto read_b = [&](int slot, uint32_t boff) __attribute__((always_inline)) {
#pragma unroll
                        for (int t = 0; t < TT; ++t) wb[slot][t] = *reinterpret_cast<const sk_u32x4*>(bl + boff + t * tile_t);
                    };
                    auto mma = [&](int sa, int sb) __attribute__((always_inline)) {
#pragma unroll
                        for (int t = 0; t < TT; ++t) {
                            acc[t][0] = sk_mfma<F16>(wa[sa][0], wb[sb][t], acc[t][0]);
                            acc[t][1] = sk_mfma<F16>(wa[sa][1], wb[sb][t], acc[t][1]);
                        }
                    };
                    req_a(0, tb[0]);
                    req_a(1, tb[2]);
                    req_a(2, tb[4]);
                    Pack<uint32_t, 2> ent = tb[6];       // entry of the step whose weights are requested next
                    stage_in(stage);
                    if constexpr (PRE) {
                        if (stage + s_step < nstages_all) stage_req(stage + s_step);
                    }
                    read_b(0, bo[0]);
                    int st = 0;
                    // Four steps per trip, no branch inside: weights three steps ahead (4 register sets), activations one step
                    // ahead (2 sets). A wave issues in order and a matrix instruction occupies the matrix pipe for 32 cycles: the
                    // requests of the coming steps are therefore spread between the matrix instructions of the current one (each
                    // gap takes a few of them for free) instead of standing in a block in front of them, where the matrix pipe
                    // would run dry while they issue.
                    auto step_order = [&]() __attribute__((always_inline)) {
                        constexpr int kMfma = 0x008, kValu = 0x002, kVmemRead = 0x020, kDsRead = 0x100;
                        __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(kValu, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(kVmemRead, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(kValu, 1, 0);
                        if constexpr (TT >= 2) {
                            __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kValu, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kValu, 1, 0);
                        }
                        if constexpr (TT >= 4) {
                            __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kValu, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kValu, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(kMfma, 2, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    };
                    for (; st + 4 <= nst_s; st += 4) {
                        req_a(3, ent);
                        ent = tb[2 * (st + 4)];
                        read_b(1, bo[1]);
                        mma(0, 0);
                        step_order();
                        req_a(0, ent);
                        ent = tb[2 * (st + 5)];
                        read_b(0, bo[2]);
                        mma(1, 1);
                        step_order();
                        req_a(1, ent);
                        ent = tb[2 * (st + 6)];
                        read_b(1, bo[3]);
                        mma(2, 0);
                        step_order();
                        req_a(2, ent);
                        ent = tb[2 * (st + 7)];
                        read_b(0, bo[0]);
                        mma(3, 1);
                        step_order();
                    }
                    // The last nst % 4 steps: wa[0..2] hold their weight fragments, wb[0] the first one's activations.
                    if (st < nst_s) {
                        if (st + 1 < nst_s) read_b(1, bo[1]);
                        mma(0, 0);
                        if (st + 1 < nst_s) {
                            if (st + 2 < nst_s) read_b(0, bo[2]);
                            mma(1, 1);
                            if (st + 2 < nst_s) mma(2, 0);
                        }
                    }
                }
            }

            // ---- epilogue. Accumulator register 4 q + k of fragment f holds channel 32 f + 8 q + 4 half + k of the lane's
            // pixel: a "quad" (f, q) is the lane's half of channel group j8 = 8 oc_tile + 4 f + q. One quad at a time: its bias
            // and membrane (4 + 4 registers) live across its timesteps; a lane's addresses are 32-bit offsets from uniform bases.
            if constexpr (!SK) {
                if (wave < 4) __builtin_amdgcn_s_setprio(0);
            }
            const float* __restrict__ v_src = t0 == 0 ? v_init : v_out;   // later windows continue from the stored membrane
            const int t_count = g.shared_x ? g.T : min(TT, g.T - t0);      // LIF steps of this window
            // (Made opaque here: everything derived from the lane's pixel offset is then computed after the matrix loop instead of
            // before it, where the compiler would otherwise park two dozen store addresses in registers or scratch memory.)
            int pxo_e = pxo, n_e = n_c, half_e = half;
            asm volatile("" : "+v"(pxo_e), "+v"(n_e), "+v"(half_e));
            const uint32_t lane_nchw = static_cast<uint32_t>((n_e * g.Cout + 4 * half_e) * po + pxo_e);        // elements
            const uint32_t lane_c8 = static_cast<uint32_t>(((n_e * g.C8out) * po + pxo_e) * 8 + 4 * half_e);   // elements
            const uint32_t lane_bits = static_cast<uint32_t>((n_e * g.C8out) * po + pxo_e);                  // bytes

            // Valid-channel mask and initial membrane of the quad of channel group j8.
            auto quad_begin = [&](int j8, float (&v)[4], uint32_t& chm) __attribute__((always_inline)) {
                const int ch0 = j8 * 8 + 4 * half_e;
                chm = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    chm |= ch0 + k < g.Cout ? (1u << k) : 0u;
                    v[k] = 0.0f;
                }
                if (v_src != nullptr && !g.analog_out && px_ok) {
                    const float* __restrict__ vp = v_src + static_cast<int64_t>(j8) * 8 * po;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if ((chm >> k) & 1u) v[k] = vp[lane_nchw + static_cast<uint32_t>(k * po)];
                }
            };
            // The residual of a quad at timestep `ta`, raw (two registers in any layout), and its addition to the quad's sums.
            auto res_load = [&](int ta, int j8, uint32_t (&raw)[2]) __attribute__((always_inline)) {
                raw[0] = 0u;
                raw[1] = 0u;
                if (g.res_layout < 0 || !(j8 < g.C8out && px_ok)) return;
                const unsigned char* __restrict__ res_t = static_cast<const unsigned char*>(sk_kernarg_ptr(kResTable, ta));
                if (g.res_layout == SNNF_LAYOUT_BITS) {
                    raw[0] = (res_t + static_cast<int64_t>(j8) * po)[lane_bits];
                } else if (g.res_layout == SNNF_LAYOUT_C8) {
                    const Pack<uint32_t, 2> r2 = *reinterpret_cast<const Pack<uint32_t, 2>*>(reinterpret_cast<const XT*>(res_t) + static_cast<int64_t>(j8) * po * 8 + lane_c8);
                    raw[0] = r2.v[0];
                    raw[1] = r2.v[1];
                } else {
                    const uint16_t* __restrict__ rp = reinterpret_cast<const uint16_t*>(res_t) + static_cast<int64_t>(j8) * 8 * po;
                    const int ch0 = j8 * 8 + 4 * half_e;
                    uint32_t e[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) e[k] = ch0 + k < g.Cout ? rp[lane_nchw + static_cast<uint32_t>(k * po)] : 0u;
                    raw[0] = e[0] | (e[1] << 16);
                    raw[1] = e[2] | (e[3] << 16);
                }
            };
            auto res_add = [&](const uint32_t (&raw)[2], float (&x)[4]) __attribute__((always_inline)) {
                if (g.res_layout < 0) return;
                if (g.res_layout == SNNF_LAYOUT_BITS) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) x[k] += ((raw[0] >> (4 * half_e + k)) & 1u) ? 1.0f : 0.0f;
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t bits = (raw[k >> 1] >> (16 * (k & 1))) & 0xffffu;
                        x[k] += to_float(XT{static_cast<uint16_t>(bits)});
                    }
                }
            };
            // Store of 4 channel values of the lane's pixel at timestep `ta` in a dense layout (C8: one 8-byte store).
            auto quad_store_dense = [&](int ta, int j8, const Pack<XT, 4>& o, uint32_t chm) __attribute__((always_inline)) {
                unsigned char* __restrict__ out_t = out + static_cast<int64_t>(ta) * g.out_step_stride;
                if (g.out_layout == SNNF_LAYOUT_C8) {
                    *reinterpret_cast<Pack<XT, 4>*>(reinterpret_cast<XT*>(out_t) + static_cast<int64_t>(j8) * po * 8 + lane_c8) = o;
                } else {
                    XT* __restrict__ op = reinterpret_cast<XT*>(out_t) + static_cast<int64_t>(j8) * 8 * po;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if ((chm >> k) & 1u) op[lane_nchw + static_cast<uint32_t>(k * po)] = o.v[k];
                }
            };
            // One step of a quad at absolute timestep `ta`: x = sums (bias included) (+ residual), then the neuron (its spikes are the
            // returned nibble) or, without a neuron, x itself written to the dense output.
            auto quad_step = [&](int ta, int j8, const float (&x_in)[4], const uint32_t (&res_raw)[2], float (&v)[4], uint32_t chm) __attribute__((always_inline)) -> uint32_t {
                const bool grp_ok = j8 < g.C8out && px_ok;
                float x[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) x[k] = x_in[k];
                res_add(res_raw, x);
                uint32_t nib = 0;
                if (!g.analog_out) {
                    if (common_lif) {   // power-of-two tau, hard reset: one test per quad step instead of two per neuron step
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            // tau = 2: (v + x) / 2, one rounding, the form the straight-line epilogue computes.
                            const float h = half_tau ? (v[k] + x[k]) * 0.5f : v[k] + (x[k] - v[k]) * lif.inv_tau;
                            const bool fired = h >= lif.v_threshold;
                            v[k] = fired ? lif.v_reset : h;
                            nib |= fired ? (1u << k) : 0u;
                        }
                    } else {
#pragma unroll
                        for (int k = 0; k < 4; ++k) nib |= lif_step(x[k], v[k], lif) ? (1u << k) : 0u;
                    }
                    nib &= chm;
                } else if (grp_ok) {
                    Pack<XT, 4> o;
#pragma unroll
                    for (int k = 0; k < 4; ++k) o.v[k] = from_float<XT>(((chm >> k) & 1u) ? x[k] : 0.0f);
                    quad_store_dense(ta, j8, o, chm);
                }
                return nib;
            };
            // Dense spike output of up to 8 consecutive steps [ta0, ta0 + cnt) of a quad from their nibbles, one step at a time
            // (a loop: dense spikes only leave at the network's boundary, and unrolled stores would cost the common path registers).
            auto quad_store_spikes = [&](int ta0, int cnt, int j8, uint32_t nibw, uint32_t chm) __attribute__((always_inline)) {
                if (j8 < g.C8out && px_ok) {
                    for (int i = 0; i < cnt; ++i) {
                        Pack<XT, 4> o;
#pragma unroll
                        for (int k = 0; k < 4; ++k) o.v[k] = spike_value<XT>((nibw >> (4 * i + k)) & 1u);
                        quad_store_dense(ta0 + i, j8, o, chm);
                    }
                }
            };
            // Bit-packed output of up to 8 consecutive steps [ta0, ta0 + cnt) of a quad: nibble i of `nibw` = step ta0 + i. The
            // other half of the wave holds the other nibble of every byte (lanes l and l + 32 own the same pixel); even
            // steps are stored by the lower half, odd steps by the upper half.
            auto quad_store_bits = [&](int ta0, int cnt, int j8, uint32_t nibw) __attribute__((always_inline)) {
                const auto both = __builtin_amdgcn_permlane32_swap(nibw, nibw, false, false);   // [0]: lanes 0..31's word, [1]: lanes 32..63's
                const uint32_t lo = both[0];
                const uint32_t hi = both[1];
                if (j8 < g.C8out && px_ok) {
                    unsigned char* __restrict__ ob = out + static_cast<int64_t>(j8) * po;
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        const int i = 2 * m + half_e;
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

            // FAST: the layer as it runs inside a network - bit-packed output, no or a bit-packed residual, the usual neuron
            // (tau = 2, hard reset to 0, a threshold whose power-of-two multiples are normal numbers), zero initial membrane,
            // one window, whole channel groups. Straight-line code.
            // The membrane is kept scaled, S_t = 2^t v_t: a step is then S += 2^(t-1) x (every scaling is exact, so S_t / 2^t
            // is bit for bit the (v + x) / 2 of the general path), a comparison against 2^t v_th and a select, and the carry of
            // the comparison is shifted into the quad's word of quiet (not fired) bits: four instructions per neuron step.
            // After n steps the word holds step i's nibble at bits [4 (n - 1 - i), +4), bit k of a nibble = neuron k.
            auto fast_step4 = [&](const float (&x)[4], int t, float (&S)[4], uint32_t& quiet) __attribute__((always_inline)) {
                const float c = __uint_as_float(static_cast<uint32_t>(127 + t) << 23);                                   // 2^t
                const float th2 = __uint_as_float(__float_as_uint(lif.v_threshold) + (static_cast<uint32_t>(t + 1) << 23));   // 2^(t+1) v_th
                // Neuron 3 first: the last bit shifted in (neuron 0) lands at the nibble's bit 0. The four comparisons write four
                // mask registers and every instruction that reads a mask stands at least two instructions behind the one that
                // wrote it (a vector instruction may not read a scalar register that the previous two vector instructions wrote).
                uint64_t m0, m1, m2, m3;
                asm("v_fmac_f32 %0, %9, %13\n\t"
                    "v_fmac_f32 %1, %9, %12\n\t"
                    "v_fmac_f32 %2, %9, %11\n\t"
                    "v_fmac_f32 %3, %9, %10\n\t"
                    "v_cmp_nle_f32_e64 %5, %14, %0\n\t"
                    "v_cmp_nle_f32_e64 %6, %14, %1\n\t"
                    "v_cmp_nle_f32_e64 %7, %14, %2\n\t"
                    "v_cmp_nle_f32_e64 %8, %14, %3\n\t"
                    "v_cndmask_b32_e64 %0, 0, %0, %5\n\t"
                    "v_cndmask_b32_e64 %1, 0, %1, %6\n\t"
                    "v_cndmask_b32_e64 %2, 0, %2, %7\n\t"
                    "v_cndmask_b32_e64 %3, 0, %3, %8\n\t"
                    "v_addc_co_u32_e64 %4, vcc, %4, %4, %5\n\t"
                    "v_addc_co_u32_e64 %4, vcc, %4, %4, %6\n\t"
                    "v_addc_co_u32_e64 %4, vcc, %4, %4, %7\n\t"
                    "v_addc_co_u32_e64 %4, vcc, %4, %4, %8"
                    : "+v"(S[3]), "+v"(S[2]), "+v"(S[1]), "+v"(S[0]), "+v"(quiet), "=&s"(m3), "=&s"(m2), "=&s"(m1), "=&s"(m0)
                    : "s"(c), "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "s"(th2)
                    : "vcc");
            };
            // x += the residual spikes of this half of the byte (bit k of the nibble -> 0.0 / 1.0 through one byte each).
            auto fast_add_res = [&](uint32_t res_byte, float (&x)[4]) __attribute__((always_inline)) {
                const uint32_t nib = (res_byte >> (4 * half_e)) & 15u;
                const uint32_t spread = __umul24(nib, 0x00204081u) & 0x01010101u;
#pragma unroll
                for (int k = 0; k < 4; ++k) x[k] += static_cast<float>((spread >> (8 * k)) & 0xffu);
            };
            // Residual byte of channel group j8 at timestep ta for this lane's pixel (this half's nibble is picked at the use,
            // so that nothing waits on the load where it is issued). Lanes without a pixel read pixel 0 of image 0 (their
            // result is never stored).
            auto fast_res = [&](int ta, int j8) __attribute__((always_inline)) -> uint32_t {
                const unsigned char* __restrict__ res_t = static_cast<const unsigned char*>(sk_kernarg_ptr(kResTable, ta));
                return (res_t + static_cast<int64_t>(min(j8, g.C8out - 1)) * po)[lane_bits];
            };
            // Bit-packed store of the n <= 8 steps [ta0, ta0 + n) of a quad from its word of quiet bits. Lanes l and l + 32 own
            // the two nibbles of every byte of a pixel and swap their words in registers; even steps are stored by the lower
            // half of the wave, odd steps by the upper half.
            auto fast_store = [&](int ta0, int n, int j8, uint32_t quiet) __attribute__((always_inline)) {
                const uint32_t fired = ~quiet;
                const auto both = __builtin_amdgcn_permlane32_swap(fired, fired, false, false);   // [0]: lanes 0..31's word, [1]: lanes 32..63's
                if (j8 < g.C8out && px_ok) {
                    unsigned char* __restrict__ ob = out + static_cast<int64_t>(j8) * po;
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        const int i = 2 * m + half_e;
                        if (i < n) {
                            const uint32_t sh = 4u * static_cast<uint32_t>(n - 1 - i);
                            const uint32_t byte = ((both[0] >> sh) & 15u) | (((both[1] >> sh) & 15u) << 4);
                            ob[static_cast<uint32_t>(ta0 + i) * static_cast<uint32_t>(g.out_step_stride) + lane_bits] = static_cast<unsigned char>(byte);
                        }
                    }
                }
            };
            // The same for exactly the four steps 0..3 (the usual window), without a condition per step: the lower half
            // stores steps 0 and 2, the upper half steps 1 and 3.
            auto fast_store4 = [&](int j8, uint32_t quiet) __attribute__((always_inline)) {
                const uint32_t fired = ~quiet;
                const auto both = __builtin_amdgcn_permlane32_swap(fired, fired, false, false);
                if (j8 < g.C8out && px_ok) {
                    unsigned char* __restrict__ ob = out + static_cast<int64_t>(j8) * po;
                    const uint32_t first = lane_bits + (half_e ? static_cast<uint32_t>(g.out_step_stride) : 0u);
                    const uint32_t sh = half_e ? 8u : 12u;
                    ob[first] = static_cast<unsigned char>(((both[0] >> sh) & 15u) | (((both[1] >> sh) & 15u) << 4));
                    ob[first + 2u * static_cast<uint32_t>(g.out_step_stride)] =
                        static_cast<unsigned char>(((both[0] >> (sh - 8u)) & 15u) | (((both[1] >> (sh - 8u)) & 15u) << 4));
                }
            };
            // The four steps 0..3 as 2x2 average pools of the spikes (POOL): the four lanes of a window (patches have even
            // extents, so a window lies inside one wave half) hold one byte-wide count per channel and step, add them in a
            // reduce-scatter of two exchanges (first with the horizontal neighbour, two steps each way; then with the vertical
            // one, one step each way), and the lane at window position (row r, column c) ends up with step 2 c + r, whose
            // four quarters it stores as 16-bit values of the pooled, channel-blocked tensor.
            auto fast_store4_pooled = [&](int j8, uint32_t quiet) __attribute__((always_inline)) {
                const uint32_t fired = ~quiet;
                uint32_t w[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) w[t] = __umul24((fired >> (4 * (3 - t))) & 15u, 0x00204081u) & 0x01010101u;
                int lane_e = lane;
                asm volatile("" : "+v"(lane_e));
                const uint32_t pos = reinterpret_cast<const uint32_t*>(lds + kSpkTableBytes + kSpkDescBytes)[lane_e & 31];
                const int pi_e = static_cast<int>(pos & 255u), prow_e = static_cast<int>((pos >> 8) & 255u), pcol_e = static_cast<int>(pos >> 16);
                const bool odd_col = (pcol_e & 1) != 0, odd_row = (prow_e & 1) != 0;
                uint32_t keep0 = odd_col ? w[2] : w[0], keep1 = odd_col ? w[3] : w[1];
                const uint32_t give0 = odd_col ? w[0] : w[2], give1 = odd_col ? w[1] : w[3];
                const int side = (lane_e ^ 1) * 4;
                keep0 += static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(side, static_cast<int>(give0)));
                keep1 += static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(side, static_cast<int>(give1)));
                uint32_t keep = odd_row ? keep1 : keep0;
                const uint32_t give = odd_row ? keep0 : keep1;
                keep += static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute((lane_e + (odd_row ? -g.PC : g.PC)) * 4, static_cast<int>(give)));
                if (j8 < g.C8out && px_ok) {
                    const int step = (odd_col ? 2 : 0) + (odd_row ? 1 : 0);
                    const int hp = g.Ho >> 1, wp = g.Wo >> 1;
                    const uint32_t off = static_cast<uint32_t>(((((n0 + pi_e) * g.C8out + j8) * hp + ((oh0 + prow_e) >> 1)) * wp + ((ow0 + pcol_e) >> 1)) * 8 + 4 * half_e);
                    Pack<XT, 4> q4;
#pragma unroll
                    for (int k = 0; k < 4; ++k) q4.v[k] = from_float<XT>(static_cast<float>((keep >> (8 * k)) & 255u) * 0.25f);
                    *reinterpret_cast<Pack<XT, 4>*>(out + static_cast<int64_t>(step) * g.out_step_stride + static_cast<int64_t>(off) * 2) = q4;
                }
            };
            // All steps of one quad whose sums are xq[tw][k]: residual, LIF, bit-packed store, optional membrane store.
            auto fast_quad = [&](int j8, const float (&xq)[TT][4], const uint32_t (&rb)[TT], bool with_res) __attribute__((always_inline)) {
                float S[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                if constexpr (TT == 1) {
                    if (t_count == 4 && !with_res) {
                        // The usual stem: one frame, four steps, no residual. Straight-line.
                        uint32_t quiet = 0;
#pragma unroll
                        for (int i = 0; i < 4; ++i) fast_step4(xq[0], i, S, quiet);
                        if constexpr (POOL) fast_store4_pooled(j8, quiet);
                        else fast_store4(j8, quiet);
                    } else {
                        for (int ta0 = 0; ta0 < t_count; ta0 += 8) {
                            const int cnt = min(8, t_count - ta0);
                            uint32_t quiet = 0;
                            for (int i = 0; i < cnt; ++i) {
                                float x[4];
#pragma unroll
                                for (int k = 0; k < 4; ++k) x[k] = xq[0][k];
                                if (with_res) fast_add_res(fast_res(ta0 + i, j8), x);
                                fast_step4(x, ta0 + i, S, quiet);
                            }
                            fast_store(ta0, cnt, j8, quiet);
                        }
                    }
                } else {
                    uint32_t quiet = 0;
                    if (t_count == TT) {
                        // Every step of the window is real (the usual case): no condition per step.
                        if (with_res) {
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw) {
                                float x[4];
#pragma unroll
                                for (int k = 0; k < 4; ++k) x[k] = xq[tw][k];
                                fast_add_res(rb[tw], x);
                                fast_step4(x, tw, S, quiet);
                            }
                        } else {
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw) fast_step4(xq[tw], tw, S, quiet);
                        }
                        if constexpr (TT == 4) {
                            if constexpr (POOL) fast_store4_pooled(j8, quiet);
                            else fast_store4(j8, quiet);
                        } else {
                            fast_store(0, TT, j8, quiet);
                        }
                    } else {
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw) {
                            if (tw < t_count) {
                                float x[4];
#pragma unroll
                                for (int k = 0; k < 4; ++k) x[k] = xq[tw][k];
                                if (with_res) fast_add_res(rb[tw], x);
                                fast_step4(x, tw, S, quiet);
                            }
                        }
                        fast_store(0, t_count, j8, quiet);
                    }
                }
                if (v_out != nullptr && px_ok && j8 < g.C8out) {
                    float* __restrict__ vp = v_out + static_cast<int64_t>(j8) * 8 * po;
                    const float unscale = __uint_as_float(static_cast<uint32_t>(127 - t_count) << 23);   // 2^-t_count
#pragma unroll
                    for (int k = 0; k < 4; ++k) vp[lane_nchw + static_cast<uint32_t>(k * po)] = S[k] * unscale;
                }
            };
            // All steps of one quad, any layouts and neuron (the general path).
            auto general_quad = [&](int j8, const float (&xq)[TT][4]) __attribute__((always_inline)) {
                float v[4];
                uint32_t chm;
                quad_begin(j8, v, chm);
                if constexpr (TT == 1) {
                    // One convolution result, t_count LIF steps on it (one step, or one frame shared by all T timesteps).
                    for (int ta0 = 0; ta0 < t_count; ta0 += 8) {
                        const int cnt = min(8, t_count - ta0);
                        uint32_t nibw = 0;
                        for (int i = 0; i < cnt; ++i) {
                            uint32_t rr[2];
                            res_load(t0 + ta0 + i, j8, rr);
                            nibw |= quad_step(t0 + ta0 + i, j8, xq[0], rr, v, chm) << (4 * i);
                        }
                        if (g.out_layout == SNNF_LAYOUT_BITS) quad_store_bits(t0 + ta0, cnt, j8, nibw);
                        else if (!g.analog_out) quad_store_spikes(t0 + ta0, cnt, j8, nibw, chm);
                    }
                } else {
                    uint32_t rr[TT][2];
#pragma unroll
                    for (int tw = 0; tw < TT; ++tw) res_load(min(t0 + tw, g.T - 1), j8, rr[tw]);
                    uint32_t nibw = 0;
#pragma unroll
                    for (int tw = 0; tw < TT; ++tw)
                        if (tw < t_count) nibw |= quad_step(t0 + tw, j8, xq[tw], rr[tw], v, chm) << (4 * tw);
                    if (g.out_layout == SNNF_LAYOUT_BITS) quad_store_bits(t0, t_count, j8, nibw);
                    else if (!g.analog_out) quad_store_spikes(t0, t_count, j8, nibw, chm);
                }
                quad_end(j8, v, chm);
            };

            if constexpr (!SK) {
                if constexpr (FAST) {
                    const bool with_res = g.res_layout >= 0;
                    // The residual bytes of all 8 quads are requested up front (the matrix loop's operand registers are free now):
                    // one round trip to memory for the whole epilogue. The fence keeps the compiler from sinking each request
                    // to its use, where every one of them would be waited for in turn.
                    uint32_t rb[8][TT];
#pragma unroll
                    for (int fq = 0; fq < 8; ++fq)
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw) rb[fq][tw] = 0u;
                    if (with_res && TT > 1) {
                        const unsigned char* res_ptr[TT];
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw)
                            res_ptr[tw] = static_cast<const unsigned char*>(sk_kernarg_ptr(kResTable, min(tw, t_count - 1))) + static_cast<int64_t>(oc_e) * 8 * po;
                        auto req_res = [&](auto fq_tag) __attribute__((always_inline)) {
                            constexpr int fq = decltype(fq_tag)::value;
                            const uint32_t off = lane_bits + static_cast<uint32_t>(min(fq, g.C8out - 1 - oc_e * 8) * po);
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw) rb[fq][tw] = res_ptr[tw][off];
                        };
                        req_res(std::integral_constant<int, 0>{});
                        req_res(std::integral_constant<int, 1>{});
                        req_res(std::integral_constant<int, 2>{});
                        req_res(std::integral_constant<int, 3>{});
                        req_res(std::integral_constant<int, 4>{});
                        req_res(std::integral_constant<int, 5>{});
                        req_res(std::integral_constant<int, 6>{});
                        req_res(std::integral_constant<int, 7>{});
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    auto do_quad = [&](auto fq_tag) __attribute__((always_inline)) {
                        constexpr int fq = decltype(fq_tag)::value;
                        float xq[TT][4];
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw)
#pragma unroll
                            for (int k = 0; k < 4; ++k) xq[tw][k] = acc[tw][fq >> 2][4 * (fq & 3) + k];
                        fast_quad(oc_e * 8 + fq, xq, rb[fq], with_res);
                    };
                    do_quad(std::integral_constant<int, 0>{});
                    do_quad(std::integral_constant<int, 1>{});
                    do_quad(std::integral_constant<int, 2>{});
                    do_quad(std::integral_constant<int, 3>{});
                    do_quad(std::integral_constant<int, 4>{});
                    do_quad(std::integral_constant<int, 5>{});
                    do_quad(std::integral_constant<int, 6>{});
                    do_quad(std::integral_constant<int, 7>{});
                } else {
                    // A runtime loop over the wave's 8 quads keeps the code small; a quad's sums are copied out of the accumulators
                    // by a switch (constant register indices), so the accumulators stay in registers.
                    for (int fq = 0; fq < 8; ++fq) {
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
                        general_quad(oc_e * 8 + fq, xq);
                    }
                }
            } else {
                // Split K: the WK waves of a tile add their partial sums through LDS (the staging regions are dead by then).
                float* __restrict__ part = reinterpret_cast<float*>(lds + kSpkHeaderBytes);      // [wave][e 0..3][tw][lane][4]
#define SNNF_SPK_PARK_QUAD(E, F)                                                                                                 \
    _Pragma("unroll") for (int tw = 0; tw < TT; ++tw) {                                                                          \
        const sk_f32x4 four = {acc[tw][F][4 * (E)], acc[tw][F][4 * (E) + 1], acc[tw][F][4 * (E) + 2], acc[tw][F][4 * (E) + 3]};  \
        *reinterpret_cast<sk_f32x4*>(part + (((wave * 4 + (E)) * TT + tw) * 64 + lane) * 4) = four;                             \
    }
                if (WK == 2) {
                    // Two waves per tile: wave wk finishes the four quads of fragment wk, which sit in the first half of its
                    // accumulators (the second wave computes the fragments in swapped places). It hands its sums of the other
                    // fragment to its partner and adds the partner's sums to its own, which never leave their registers: one exchange.
                    __syncthreads();   // every wave is done with its staging region
                    SNNF_SPK_PARK_QUAD(0, 1) SNNF_SPK_PARK_QUAD(1, 1) SNNF_SPK_PARK_QUAD(2, 1) SNNF_SPK_PARK_QUAD(3, 1)
                    uint32_t rb[TT];
#pragma unroll
                    for (int tw = 0; tw < TT; ++tw) rb[tw] = 0u;
                    if constexpr (FAST) {   // the residual bytes of the first quad travel while the workgroup meets
                        if (g.res_layout >= 0 && TT > 1) {
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw) rb[tw] = fast_res(min(tw, t_count - 1), oc_e * 8 + 4 * wk);
                        }
                    }
                    __syncthreads();
                    const int partner = wave ^ 1;
                    int lane_x = lane;                   // opaque: the addresses below are computed here, not ahead of the matrix loop
                    asm volatile("" : "+v"(lane_x));
                    for (int e = 0; e < 4; ++e) {
                        const int j8 = oc_e * 8 + 4 * wk + e;
                        sk_f32x4 theirs[TT];
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw)
                            theirs[tw] = *reinterpret_cast<const sk_f32x4*>(part + (((partner * 4 + e) * TT + tw) * 64 + lane_x) * 4);
                        float xq[TT][4];
#define SNNF_SPK_COPY_QUAD(F, Q)                                          \
    _Pragma("unroll") for (int tw = 0; tw < TT; ++tw)                     \
        _Pragma("unroll") for (int k = 0; k < 4; ++k) xq[tw][k] = acc[tw][F][4 * (Q) + k]
                        switch (e) {
                            case 0: SNNF_SPK_COPY_QUAD(0, 0); break;
                            case 1: SNNF_SPK_COPY_QUAD(0, 1); break;
                            case 2: SNNF_SPK_COPY_QUAD(0, 2); break;
                            default: SNNF_SPK_COPY_QUAD(0, 3); break;
                        }
#undef SNNF_SPK_COPY_QUAD
#pragma unroll
                        for (int tw = 0; tw < TT; ++tw)
#pragma unroll
                            for (int k = 0; k < 4; ++k) xq[tw][k] += theirs[tw][k];   // a sum of two terms: the same in either order
                        if constexpr (FAST) {
                            if (e != 0 && g.res_layout >= 0 && TT > 1) {
#pragma unroll
                                for (int tw = 0; tw < TT; ++tw) rb[tw] = fast_res(min(tw, t_count - 1), j8);
                            }
                            fast_quad(j8, xq, rb, g.res_layout >= 0);
                        } else {
                            general_quad(j8, xq);
                        }
                    }
                } else
                // More waves per tile: four quads per round for all TT timesteps; quad 4 r + e of round r is finished by wave
                // (4 r + e) mod WK of the tile, which adds the WK partial sums in a fixed order and then runs that quad's timesteps
                // like the unsplit kernel.
                for (int r = 0; r < 2; ++r) {
                    __syncthreads();   // the previous round's sums are consumed (first round: every wave is done with its staging region)
                    if (r == 0) {
                        SNNF_SPK_PARK_QUAD(0, 0) SNNF_SPK_PARK_QUAD(1, 0) SNNF_SPK_PARK_QUAD(2, 0) SNNF_SPK_PARK_QUAD(3, 0)
                    } else {
                        SNNF_SPK_PARK_QUAD(0, 1) SNNF_SPK_PARK_QUAD(1, 1) SNNF_SPK_PARK_QUAD(2, 1) SNNF_SPK_PARK_QUAD(3, 1)
                    }
#undef SNNF_SPK_PARK_QUAD
                    const int e_first = (wk - 4 * r) & (WK - 1);      // this wave finishes quads 4 r + e, e = e_first, e_first + WK, ... < 4
                    // The residual bytes of the wave's first quad travel while the workgroup meets.
                    uint32_t rb[TT];
#pragma unroll
                    for (int tw = 0; tw < TT; ++tw) rb[tw] = 0u;
                    if constexpr (FAST) {
                        if (e_first < 4 && g.res_layout >= 0 && TT > 1) {
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw) rb[tw] = fast_res(min(tw, t_count - 1), oc_e * 8 + 4 * r + e_first);
                        }
                    }
                    __syncthreads();
                    for (int e_own = e_first; e_own < 4; e_own += WK) {
                        const int j8 = oc_e * 8 + 4 * r + e_own;
                        float xq[TT][4];
                        {
                            // The partial sums of the tile's waves, all timesteps of a wave (of two waves) in flight together (WK is a power
                            // of two >= 2); added in the order of the waves.
                            sk_f32x4 sum[TT];
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw) sum[tw] = sk_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                            if constexpr (FAST) {
                                for (int k = 0; k < WK; k += 2) {
                                    sk_f32x4 p0[TT], p1[TT];
#pragma unroll
                                    for (int tw = 0; tw < TT; ++tw) {
                                        p0[tw] = *reinterpret_cast<const sk_f32x4*>(part + ((((tile_in_block * WK + k) * 4 + e_own) * TT + tw) * 64 + lane) * 4);
                                        p1[tw] = *reinterpret_cast<const sk_f32x4*>(part + ((((tile_in_block * WK + k + 1) * 4 + e_own) * TT + tw) * 64 + lane) * 4);
                                    }
#pragma unroll
                                    for (int tw = 0; tw < TT; ++tw) sum[tw] = (sum[tw] + p0[tw]) + p1[tw];
                                }
                            } else {   // the general epilogue has no registers to spare: one wave's sums at a time
                                for (int k = 0; k < WK; ++k) {
#pragma unroll
                                    for (int tw = 0; tw < TT; ++tw)
                                        sum[tw] += *reinterpret_cast<const sk_f32x4*>(part + ((((tile_in_block * WK + k) * 4 + e_own) * TT + tw) * 64 + lane) * 4);
                                }
                            }
#pragma unroll
                            for (int tw = 0; tw < TT; ++tw)
#pragma unroll
                                for (int k = 0; k < 4; ++k) xq[tw][k] = sum[tw][k];
                        }
                        if constexpr (FAST) {
                            if (e_own != e_first && g.res_layout >= 0 && TT > 1) {
#pragma unroll
                                for (int tw = 0; tw < TT; ++tw) rb[tw] = fast_res(min(tw, t_count - 1), j8);
                            }
                            fast_quad(j8, xq, rb, g.res_layout >= 0);
                        } else {
                            general_quad(j8, xq);
                        }
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
                                                                        static_cast<unsigned char*>(L.out), L.v_out, L.lif, L.wpacked2, L.bias2);
        return check_launch("snnf_conv_lif_blocked");
    };
    if (L.fast_epilogue) return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, TT, IN, true, true>) : run(conv_spk_kernel<XT, TT, IN, false, true>);
    return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, TT, IN, true, false>) : run(conv_spk_kernel<XT, TT, IN, false, false>);
}

// The variants whose spikes leave as 2x2 average pools: straight-line epilogue, four steps (side by side, or of one frame).
template <typename XT, int IN>
int launch_conv_spk_pooled(const SpkLaunch& L, int tt) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif_blocked_avgpool"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kSpkWaves * 64, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.g, L.wpacked, L.bias, L.v_init,
                                                                        static_cast<unsigned char*>(L.out), L.v_out, L.lif, L.wpacked2, L.bias2);
        return check_launch("snnf_conv_lif_blocked_avgpool");
    };
    if (tt == 4) return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 4, IN, true, true, false, true>) : run(conv_spk_kernel<XT, 4, IN, false, true, false, true>);
    return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 1, IN, true, true, false, true>) : run(conv_spk_kernel<XT, 1, IN, false, true, false, true>);
}

// The variants that read the network's input as it is: one dense frame of at most 8 channels for all timesteps.
template <typename XT>
int launch_conv_spk_frame(const SpkLaunch& L, bool pooled) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif_blocked"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kSpkWaves * 64, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.g, L.wpacked, L.bias, L.v_init,
                                                                        static_cast<unsigned char*>(L.out), L.v_out, L.lif, L.wpacked2, L.bias2);
        return check_launch("snnf_conv_lif_blocked");
    };
    constexpr int D = SNNF_LAYOUT_NCHW;
    if (pooled) return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 1, D, true, true, false, true>) : run(conv_spk_kernel<XT, 1, D, false, true, false, true>);
    if (L.fast_epilogue) return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 1, D, true, true>) : run(conv_spk_kernel<XT, 1, D, false, true>);
    return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 1, D, true, false>) : run(conv_spk_kernel<XT, 1, D, false, false>);
}

// The variants with a projection shortcut in the accumulators: bit-packed inputs, four timesteps side by side.
template <typename XT>
int launch_conv_spk_shortcut(const SpkLaunch& L) {
    auto run = [&](auto kernel) -> int {
        if (const int rc = reserve_lds(reinterpret_cast<const void*>(kernel), L.lds_bytes, "snnf_conv_lif_blocked_shortcut"); rc != SNNF_OK) return rc;
        kernel<<<dim3(L.grid), kSpkWaves * 64, L.lds_bytes, L.stream>>>(L.xs, L.residuals, L.g, L.wpacked, L.bias, L.v_init,
                                                                        static_cast<unsigned char*>(L.out), L.v_out, L.lif, L.wpacked2, L.bias2);
        return check_launch("snnf_conv_lif_blocked_shortcut");
    };
    constexpr int B = SNNF_LAYOUT_BITS;
    if (L.fast_epilogue) return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 4, B, true, true, true>) : run(conv_spk_kernel<XT, 4, B, false, true, true>);
    return L.g.wk_log2 > 0 ? run(conv_spk_kernel<XT, 4, B, true, false, true>) : run(conv_spk_kernel<XT, 4, B, false, false, true>);
}

template <typename XT, int IN>
int launch_conv_spk_tt(const SpkLaunch& L, int tt) {
    if (tt == 4) return launch_conv_spk_variant<XT, 4, IN>(L);
    if (tt == 2) return launch_conv_spk_variant<XT, 2, IN>(L);
    return launch_conv_spk_variant<XT, 1, IN>(L);
}

// One launcher per activation dtype and input layout (each in its own translation unit, so that they compile in parallel).
int launch_conv_spk_bf16_bits(const SpkLaunch& L, int tt);
int launch_conv_spk_bf16_c8(const SpkLaunch& L, int tt);
int launch_conv_spk_f16_bits(const SpkLaunch& L, int tt);
int launch_conv_spk_f16_c8(const SpkLaunch& L, int tt);
int launch_conv_spk_bf16_shortcut(const SpkLaunch& L);
int launch_conv_spk_f16_shortcut(const SpkLaunch& L);
int launch_conv_spk_bf16_pooled(const SpkLaunch& L, int tt);
int launch_conv_spk_f16_pooled(const SpkLaunch& L, int tt);
int launch_conv_spk_bf16_frame(const SpkLaunch& L, bool pooled);
int launch_conv_spk_f16_frame(const SpkLaunch& L, bool pooled);

}  // namespace snnf
