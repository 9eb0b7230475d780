// Geometry shared by the weight packer, the tile planner and the implicit-GEMM conv+LIF kernel.
#pragma once

#include "snnf_common.h"

#include <mutex>
#include <set>
#include <utility>

namespace snnf {

constexpr int kConvThreads = 256;   // 4 waves
constexpr int kFragBytes = 1024;    // one packed 32(oc) x 16(k) weight fragment: 64 lanes x 16 bytes
constexpr int kNPF = 2;             // pixel fragments per wave: a lane owns 2 adjacent output pixels
constexpr int kNOF = 2;             // output-channel fragments per wave (64 channels)
constexpr int kMaxItems = 8;        // staging items (8 channels x 2 pixels) per thread and channel chunk
constexpr size_t kMaxLds = 160 * 1024;
constexpr int kEpiPitch = 68;       // floats per channel row of the epilogue stage (64 pixels + padding)
constexpr size_t kToutStageBytes = 4 * 64 * 12 * sizeof(float);   // time-outer kernel: four waves x 64 pixels x (8 rows + padding)
constexpr size_t kPwStageBytes = 4 * 8 * 68 * sizeof(float);      // pointwise kernel: four waves x 8 channel rows x (64 pixels + padding)
constexpr size_t kMmBiasBytes = 512 * sizeof(float) + 16;             // matrix kernel: the workgroup's bias values (at most 8 waves x 64 channels) + one flag word
constexpr size_t kMmStageBytesPerWave = 16 * 40 * sizeof(float);  // matrix kernel, per wave: 16 channel rows x (32 pixels + padding)
constexpr size_t kEpiBytes = 4 * 4 * 8 * kEpiPitch * sizeof(float);  // four waves x (up to 4 steps x 8 channel rows)

// Channels per chunk staged in LDS; fixed by (Cin, taps, activation width) alone so that packing and the kernel agree.
// Pointwise convolutions take up to 128 channels at a time (no halo re-use to pay for), everything else 32; fp32
// activations need two prefetch registers per fetch and therefore use chunks of half the size.
__host__ __device__ inline int chunk_channels(int Cin, int taps, bool wide_activations) {
    if (Cin <= 8) return 8;
    if (Cin <= 16) return 16;
    if (taps > 1) return wide_activations ? 16 : 32;
    if (Cin <= 32) return 32;
    if (Cin <= 64 || wide_activations) return 64;
    return 128;
}

// fp32 tensors keep (nearly) fp32 accuracy on the 16-bit matrix cores by a split of both operands into two bf16 terms,
// x = x_hi + x_lo and w = w_hi + w_lo (hi = the value rounded to bf16, lo = the remainder rounded to bf16), and three of the
// four products: w_hi x_hi + w_lo x_hi + w_hi x_lo (the fourth is below 2^-16 of the result). The three products are three
// "parts" of the channel axis: the packed weight holds the real channel chunks three times over (w_hi, w_lo, w_hi) and the
// kernels stage the real activation chunks three times (x_hi, x_hi, x_lo). 16-bit tensors have one part.
constexpr int kSplitParts = 3;

struct PackGeom {
    int Cout, Cin, KH, KW;
    int CK, nchunks, npairs, nocf;
    int nchunks_r;   // real channel chunks; nchunks = parts * nchunks_r
};

__host__ __device__ inline PackGeom make_pack_geom(int Cout, int Cin, int KH, int KW, bool wide_activations) {
    PackGeom p;
    p.Cout = Cout;
    p.Cin = Cin;
    p.KH = KH;
    p.KW = KW;
    p.CK = chunk_channels(Cin, KH * KW, wide_activations);
    p.nchunks_r = (Cin + p.CK - 1) / p.CK;
    p.nchunks = (wide_activations ? kSplitParts : 1) * p.nchunks_r;
    const int slots = KH * KW * (p.CK / 8);
    p.npairs = (slots + 1) / 2;
    p.nocf = (Cout + 31) / 32;
    return p;
}

// 16-bit elements of the packed weight: [oc fragment][channel chunk][slot pair][lane 0..63][8]; fp32 bias follows.
// Slot s of a chunk = tap * (CK / 8) + channel group; pair p holds slots 2p (lanes 0-31) and 2p + 1 (lanes 32-63).
__host__ __device__ inline size_t packed_weight_elems(const PackGeom& p) {
    return static_cast<size_t>(p.nocf) * p.nchunks * p.npairs * (kFragBytes / 2);
}

// fp32 bias values behind the packed weight: zero beyond Cout, padded to whole tiles of 64 channels and followed by 64 more
// zeros (kernels read a tile's bias, or "no bias", without a bounds check).
__host__ __device__ inline size_t packed_bias_floats(const PackGeom& p) { return static_cast<size_t>((p.nocf + 1) / 2) * 64 + 64; }

// How activations are fetched from global memory while staging: two adjacent pixels of one channel per fetch.
enum LoadMode : int {
    LOAD_PAIR32 = 0,   // 16-bit activations, pixel pairs 4-byte aligned: one dword load
    LOAD_2X16 = 1,     // 16-bit activations, unaligned: two halfword loads
    LOAD_2XF32 = 2,    // fp32 activations: two dword loads, rounded to bf16 on the way into LDS
    LOAD_ROWBITS = 3   // row-packed spikes (one byte = 8 consecutive pixels of a channel): one byte load, the pair's two bits
                       // become two 16-bit ones or zeros on the way into LDS (pointwise kernel only)
};

// Part (0, 1, 2) and real channel chunk of virtual chunk `vchunk` of an fp32 tensor's three-part channel axis.
__device__ __forceinline__ void split_chunk(int vchunk, int nchunks_r, int& part, int& chunk) {
    part = vchunk >= 2 * nchunks_r ? 2 : (vchunk >= nchunks_r ? 1 : 0);
    chunk = vchunk - part * nchunks_r;
}

// Staging items a thread may hold in flight per chunk: modes that need two registers per fetch get half as many.
__host__ __device__ constexpr int staging_items(int load_mode) { return load_mode == LOAD_PAIR32 ? kMaxItems : kMaxItems / 2; }

// Division by a divisor fixed at launch as a multiply-high and a shift (the divisions of the tile walk are otherwise
// ~40-instruction sequences on the vector unit). Exact for numerators below 2^31.
struct FastDiv {
    uint32_t mul;     // 0: the divisor is 1
    uint32_t shift;
    uint32_t d;
};

inline FastDiv make_fast_div(int divisor) {
    FastDiv f;
    f.d = static_cast<uint32_t>(divisor < 1 ? 1 : divisor);
    f.mul = 0;
    f.shift = 0;
    if (f.d > 1) {
        uint32_t lg = 0;
        while ((1ull << lg) < f.d) ++lg;
        const uint32_t p = 31 + lg;
        f.mul = static_cast<uint32_t>(((1ull << p) + f.d - 1) / f.d);
        f.shift = p - 32;
    }
    return f;
}

__device__ __forceinline__ int fast_div(int n, const FastDiv& f) {
    return f.mul == 0 ? n : static_cast<int>(__umulhi(static_cast<uint32_t>(n), f.mul) >> f.shift);
}

struct ConvGeom {
    int N, Cin, H, W, Cout, KH, KW, sh, sw, ph, pw, Ho, Wo;
    int TH, TW;               // output tile: TH rows of the flattened (n, oh) row space x TW columns
    int tiles_x, tiles_y;     // ceil(Wo / TW), ceil(N * Ho / TH)
    int wm_log2, wn_log2;     // waves along pixels / along output channels (WM * WN == 4)
    int oc_tiles;             // ceil(Cout / (WN * 64))
    int CK, nchunks, npairs, groups_log2;
    int nchunks_r;            // real channel chunks of the activations (nchunks counts the three parts of an fp32 tensor)
    int NR, WT;               // LDS tile: input rows x input columns (per timestep)
    int pitch;                // bytes per LDS pixel = CK * 2 + 16
    int T;                    // timesteps stored by this launch (<= TT)
    int shared_x;             // every timestep reads the same activation tensor: convolve once
    int vec8;                 // runs of 8 output pixels may be stored as one 16-byte-aligned vector
    int64_t spike_step_stride;
    int v_is_f32;             // membrane dtype in memory: fp32 (1) or the activation dtype (0)
    int analog_out;         // matrix kernel: write conv + bias (+ residual) instead of spikes, no membrane
    int TI, img_groups;      // matrix kernel: images per tile (> 1 only when a tile is a whole output plane), ceil(N / TI)
    int w_lds;                // time-outer kernels: weight fragments streamed from L2 (0), kept in LDS (1) or in registers (2)
    int x_bufs;               // pointwise kernel: activation stages held in LDS (2 = double buffered)
    int px_base;              // pointwise kernel: pixel of each image at which this launch's tile 0 starts
    int oc_major;             // matrix kernel: an XCD takes the output-channel tiles congruent to it (all pixel tiles) instead of the pixel
                              // tiles congruent to it (all output-channel tiles); d_oc_tiles then divides by oc_tiles / 8
    int stream_out;           // pointwise kernel: spikes and membrane are stored non-temporally (the launch writes more than the caches hold)
    int bits_out;             // pointwise kernel: spikes leave row-packed (bytes), spike_step_stride counts bytes, v_out may be null
    int tiles_img;            // matrix kernel: tiles per image (tiles_x * tiles_y, tiles never straddle images)
    int run8;                 // matrix kernel: runs of 8 tile pixels are contiguous in memory and aligned for 16-byte
                              // (8) or 8-byte (4) spike accesses; 0: neither
    int wk_log2;              // matrix kernel: waves that split K of one output tile
    int mm_stage_off;         // matrix kernel: LDS offset of the waves' epilogue stages
    int stage_chunks;         // matrix kernel: packed channel chunks held by one LDS stage (pitch = stage_chunks * CK * 2 + 16)
    FastDiv d_TW, d_Ho, d_H, d_WTP, d_stage_rows, d_tiles_x, d_oc_tiles;   // d_stage_rows: NR * (WT / 2)
    FastDiv d_tiles_img, d_KW, d_npairs;
    FastDiv d_NR, d_tile_px;                                               // matrix kernel: halo rows per image, TH * TW
};

struct ConvLaunch {
    StepPtrs xs;
    StepPtrs residuals;
    int has_residual;
    ConvGeom g;
    const uint16_t* wpacked;
    const float* bias;
    const void* v_init;
    void* spikes;
    void* v_out;
    LifParams lif;
    int grid;
    size_t lds_bytes;
    hipStream_t stream;
};

// Lets `kernel` use more than 64 KiB of dynamic LDS. The attribute belongs to one kernel function on one device, so
// what has been raised already is remembered per (function, device).
inline int reserve_lds(const void* kernel, size_t bytes, const char* who) {
    if (bytes <= 64 * 1024) return SNNF_OK;
    static std::mutex mu;
    static std::set<std::pair<const void*, int>> raised;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const std::pair<const void*, int> key(kernel, dev);
    {
        std::lock_guard<std::mutex> lock(mu);
        if (raised.count(key)) return SNNF_OK;
    }
    const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
    if (err != hipSuccess) return fail(SNNF_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS: %s", who, bytes, hipGetErrorString(err));
    std::lock_guard<std::mutex> lock(mu);
    raised.insert(key);
    return SNNF_OK;
}

// One launcher per activation dtype (each in its own translation unit so they compile in parallel).
// tt: 1, 2, 4 = timesteps accumulated side by side (4-wave kernel); 10 + tt / 20 + tt = 8-wave matrix kernel, general /
// fast; 0 = time-outer kernel; -1 / -2 = pointwise kernel, general / fast.
int launch_conv_f32(const ConvLaunch& L, int tt, int load_mode);
int launch_conv_bf16(const ConvLaunch& L, int tt, int load_mode);
int launch_conv_f16(const ConvLaunch& L, int tt, int load_mode);
// Matrix kernel with 4-wave workgroups (fast variant, shared input frame: tt == 1): separate translation units.
int launch_conv_mm_w4_f32(const ConvLaunch& L, int tt, int load_mode);
int launch_conv_mm_w4_bf16(const ConvLaunch& L, int tt, int load_mode);
int launch_conv_mm_w4_f16(const ConvLaunch& L, int tt, int load_mode);

}  // namespace snnf
