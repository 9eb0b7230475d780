// Dense convolution + bias (+ residual) + LIF over T timesteps as an implicit GEMM on the gfx950 matrix cores.
//
//   out^T[Cout, T * pixels] = Wp[Cout, K] . im2col(x)[K, T * pixels],   K = taps * Cin,   then LIF along T per neuron.
//
// Mapping (v_mfma_f32_32x32x16, fp32 accumulate):
//   * M = output channels (A operand = weights), N = output pixels (B operand = activations): a lane of the result
//     owns one pixel and 16 channels per fragment, so the 32 lanes of a half wave store 32 consecutive pixels of one
//     channel plane (NCHW output).
//   * All T timesteps of a pixel tile are accumulated in the same workgroup: one weight fragment load feeds T matrix
//     operations and the LIF recurrence runs in the epilogue on accumulators that never leave registers.
//   * Weights are pre-packed (snnf_conv_pack_weight) in fragment order, so a 32x16 weight fragment is one contiguous
//     1 KiB global load straight into registers; the packed weights of a layer stay L2 resident.
//   * Activations (NCHW, pixel-contiguous) are transposed on the way into LDS to [pixel][channel] with 8 channels per
//     16-byte group, which is the per-lane operand order of the matrix instruction; a 3x3 (or any kh x kw) halo tile is
//     staged once per channel chunk and re-read for every tap with a different per-lane pixel offset. Padding and
//     image borders are handled by redirecting the lane to a zero pixel.
#include "snnf_common.h"

#include <map>
#include <mutex>
#include <tuple>

namespace snnf {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kTilePixels = 128;  // output pixels per workgroup: one 32-pixel fragment per wave
constexpr int kFragBytes = 1024;  // one packed 32(oc) x 16(k) weight fragment

// Channels per chunk staged in LDS; fixed by Cin alone so that packing and the kernel agree.
inline int chunk_channels(int Cin) { return Cin <= 8 ? 8 : (Cin <= 16 ? 16 : 32); }

struct PackGeom {
    int Cout, Cin, KH, KW;
    int CK, nchunks, npairs, nocf;
};

inline PackGeom make_pack_geom(int Cout, int Cin, int KH, int KW) {
    PackGeom p;
    p.Cout = Cout;
    p.Cin = Cin;
    p.KH = KH;
    p.KW = KW;
    p.CK = chunk_channels(Cin);
    p.nchunks = (Cin + p.CK - 1) / p.CK;
    const int slots = KH * KW * (p.CK / 8);
    p.npairs = (slots + 1) / 2;
    p.nocf = (Cout + 31) / 32;
    return p;
}

__host__ __device__ inline size_t packed_weight_elems(const PackGeom& p) {
    return static_cast<size_t>(p.nocf) * p.nchunks * p.npairs * (kFragBytes / 2);
}

// Packed layout: [oc fragment][channel chunk][slot pair][lane 0..63][8 x 16-bit], then fp32 bias[nocf * 32].
// Slot s of a chunk = tap * (CK / 8) + channel group; pair p holds slots 2p (lanes 0-31) and 2p + 1 (lanes 32-63).
template <typename WT, bool TO_F16>
__global__ void pack_weight_kernel(const WT* __restrict__ w, const WT* __restrict__ bias, PackGeom p,
                                   uint16_t* __restrict__ packed, float* __restrict__ bias_out) {
    const int64_t total = static_cast<int64_t>(packed_weight_elems(p));
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx < total) {
        const int j = idx & 7;
        const int lane = (idx >> 3) & 63;
        int64_t frag = idx >> 9;
        const int pair = frag % p.npairs;
        frag /= p.npairs;
        const int chunk = frag % p.nchunks;
        const int ocf = frag / p.nchunks;
        const int oc = ocf * 32 + (lane & 31);
        const int slot = pair * 2 + (lane >> 5);
        const int groups = p.CK / 8;
        const int tap = slot / groups;
        const int ci = chunk * p.CK + (slot % groups) * 8 + j;
        float v = 0.0f;
        if (oc < p.Cout && ci < p.Cin && tap < p.KH * p.KW)
            v = to_float(w[(static_cast<int64_t>(oc) * p.Cin + ci) * (p.KH * p.KW) + tap]);
        packed[idx] = TO_F16 ? static_cast<uint16_t>(float_to_f16_bits(v)) : static_cast<uint16_t>(float_to_bf16_bits(v));
    }
    if (idx < p.nocf * 32) bias_out[idx] = (bias != nullptr && idx < p.Cout) ? to_float(bias[idx]) : 0.0f;
}

struct ConvGeom {
    int N, Cin, H, W, Cout, KH, KW, sh, sw, ph, pw, Ho, Wo;
    int TH, TW;            // output tile: TH rows of the flattened (n, oh) row space x TW columns, TH * TW <= 128
    int tiles_x, tiles_y;  // ceil(Wo / TW), ceil(N * Ho / TH)
    int oc_tiles;          // ceil(Cout / (32 * NOF))
    int CK, nchunks, npairs, groups_log2;
    int NR, WT;            // LDS tile: input rows x input columns (per timestep)
    int pitch;             // bytes per LDS pixel = CK * 2 + 16
    int pair_aligned;      // column pairs are 4-byte aligned in global memory (2-byte activations)
    int T;                 // timesteps stored by this launch (<= TT)
    int shared_x;          // every timestep reads the same activation tensor: convolve once
    int64_t spike_step_stride;
};

template <typename XT> __device__ __forceinline__ uint32_t to_operand_bits(XT v);
template <> __device__ __forceinline__ uint32_t to_operand_bits<float>(float v) { return float_to_bf16_bits(v); }
template <> __device__ __forceinline__ uint32_t to_operand_bits<bf16_t>(bf16_t v) { return v.bits; }
template <> __device__ __forceinline__ uint32_t to_operand_bits<f16_t>(f16_t v) { return v.bits; }

template <bool F16>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

template <typename XT, typename VT, int TT, int NOF>
__global__ __launch_bounds__(kThreads) void conv_lif_kernel(StepPtrs xs, StepPtrs residuals, int has_residual,
                                                            ConvGeom g, const uint16_t* __restrict__ wpacked,
                                                            const float* __restrict__ bias,
                                                            const VT* __restrict__ v_init, XT* __restrict__ spikes,
                                                            VT* __restrict__ v_out, LifParams lif) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr bool F16 = dtype_of<XT>::value == SNNF_F16;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int half = lane >> 5;

    // ---- workgroup -> tile, keeping the workgroups that share a pixel tile on one XCD (8 XCDs, round-robin dispatch).
    const int nb = gridDim.x;
    const int q8 = nb >> 3, r8 = nb & 7;
    const int xcd = blockIdx.x & 7, slot_in_xcd = blockIdx.x >> 3;
    const int lin = xcd < r8 ? xcd * (q8 + 1) + slot_in_xcd : r8 * (q8 + 1) + (xcd - r8) * q8 + slot_in_xcd;
    const int oc_tile = lin % g.oc_tiles;
    const int px_tile = lin / g.oc_tiles;
    const int tile_x = px_tile % g.tiles_x;
    const int tile_y = px_tile / g.tiles_x;
    const int q0 = tile_y * g.TH;   // first flattened output row (n * Ho + oh)
    const int c0 = tile_x * g.TW;   // first output column
    const int total_rows = g.N * g.Ho;
    const int q_last = min(q0 + g.TH, total_rows) - 1;

    // ---- LDS tile geometry (global input row id = n * H + ih).
    const int n_first = q0 / g.Ho;
    const int g_lo = n_first * g.H + (q0 - n_first * g.Ho) * g.sh - g.ph;
    const int n_last = q_last / g.Ho;
    const int g_hi = n_last * g.H + (q_last - n_last * g.Ho) * g.sh - g.ph + g.KH - 1;
    const int rows = g_hi - g_lo + 1;  // <= g.NR by construction on the host
    int iw_lo = c0 * g.sw - g.pw;
    if (g.pair_aligned && (iw_lo & 1)) iw_lo -= 1;
    const int tile_bytes = g.NR * g.WT * g.pitch;
    const int t_in = g.shared_x ? 1 : TT;
    const int zero_off = t_in * tile_bytes;

    if (tid < g.pitch / 4) reinterpret_cast<uint32_t*>(lds + zero_off)[tid] = 0u;

    // ---- this lane's output pixel.
    const int pix = wave * 32 + (lane & 31);
    const int pr = pix / g.TW;
    const int pc = pix - pr * g.TW;
    const int q = q0 + pr;
    const int ow = c0 + pc;
    const bool pix_valid = pr < g.TH && q < total_rows && ow < g.Wo;
    const int n = pix_valid ? q / g.Ho : 0;
    const int oh = pix_valid ? q - n * g.Ho : 0;
    const int ih0 = oh * g.sh - g.ph;
    const int iw0 = ow * g.sw - g.pw;
    const int lrow0 = n * g.H + ih0 - g_lo;  // LDS row of tap kh = 0
    const int lcol0 = iw0 - iw_lo;           // LDS column of tap kw = 0
    const int groups = 1 << g.groups_log2;

    f32x16 acc[TT][NOF];
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int f = 0; f < NOF; ++f)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][f][r] = 0.0f;

    const int ocf0 = oc_tile * NOF;
    const int nocf = (g.Cout + 31) >> 5;
    const int64_t frag_stride_ocf = static_cast<int64_t>(g.nchunks) * g.npairs * (kFragBytes / 2);  // 16-bit elements

    const int WTP = g.WT >> 1;
    const int items_per_t = groups * rows * WTP;

    for (int chunk = 0; chunk < g.nchunks; ++chunk) {
        __syncthreads();  // all waves finished reading the previous chunk
        // ---- stage activations: item = (t, channel group of 8, input row, column pair) -> two 16-byte LDS pixels.
        for (int item = tid; item < t_in * items_per_t; item += kThreads) {
            const int t = item / items_per_t;
            int rem = item - t * items_per_t;
            const int cg = rem / (rows * WTP);
            rem -= cg * (rows * WTP);
            const int r = rem / WTP;
            const int cp = rem - r * WTP;
            const int grow = g_lo + r;
            const int iw = iw_lo + cp * 2;
            u32x4 lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
            if (grow >= 0 && grow < g.N * g.H) {
                const int xn = grow / g.H;
                const int ih = grow - xn * g.H;
                const bool ok0 = iw >= 0 && iw < g.W;
                const bool ok1 = iw + 1 >= 0 && iw + 1 < g.W;
                const int ci0 = chunk * g.CK + cg * 8;
                const XT* __restrict__ src =
                    static_cast<const XT*>(xs.p[t]) + ((static_cast<int64_t>(xn) * g.Cin + ci0) * g.H + ih) * g.W + iw;
                const int64_t plane = static_cast<int64_t>(g.H) * g.W;
                uint32_t e0[8], e1[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const bool cok = ci0 + j < g.Cin;
                    if constexpr (sizeof(XT) == 2) {
                        if (g.pair_aligned) {
                            const uint32_t d = (cok && ok0) ? *reinterpret_cast<const uint32_t*>(src + j * plane) : 0u;
                            e0[j] = d & 0xffffu;
                            e1[j] = d >> 16;
                        } else {
                            e0[j] = (cok && ok0) ? to_operand_bits<XT>(src[j * plane]) : 0u;
                            e1[j] = (cok && ok1) ? to_operand_bits<XT>(src[j * plane + 1]) : 0u;
                        }
                    } else {
                        e0[j] = (cok && ok0) ? to_operand_bits<XT>(src[j * plane]) : 0u;
                        e1[j] = (cok && ok1) ? to_operand_bits<XT>(src[j * plane + 1]) : 0u;
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    lo[k] = e0[2 * k] | (e0[2 * k + 1] << 16);
                    hi[k] = e1[2 * k] | (e1[2 * k + 1] << 16);
                }
            }
            unsigned char* dst = lds + t * tile_bytes + (r * g.WT + cp * 2) * g.pitch + cg * 16;
            *reinterpret_cast<u32x4*>(dst) = lo;
            *reinterpret_cast<u32x4*>(dst + g.pitch) = hi;
        }
        __syncthreads();

        // ---- matrix work for this chunk: slot s = 2 * pair + half -> (tap, channel group).
        int cg = half & (groups - 1);
        int tap_adv = half >> g.groups_log2;  // taps to advance before the first pair (1 only when groups == 1)
        int kh = 0, kw = 0;
        if (tap_adv) { kw = 1; if (kw == g.KW) { kw = 0; kh = 1; } }
        const uint16_t* __restrict__ wbase = wpacked + static_cast<int64_t>(chunk) * g.npairs * (kFragBytes / 2) + lane * 8;
        for (int pair = 0; pair < g.npairs; ++pair) {
            u32x4 a[NOF];
#pragma unroll
            for (int f = 0; f < NOF; ++f) {
                const int ocf = min(ocf0 + f, nocf - 1);
                a[f] = *reinterpret_cast<const u32x4*>(wbase + ocf * frag_stride_ocf + static_cast<int64_t>(pair) * (kFragBytes / 2));
            }
            const bool ok = pix_valid && kh < g.KH && static_cast<unsigned>(ih0 + kh) < static_cast<unsigned>(g.H) &&
                            static_cast<unsigned>(iw0 + kw) < static_cast<unsigned>(g.W);
            const int off = ok ? ((lrow0 + kh) * g.WT + lcol0 + kw) * g.pitch + cg * 16 : zero_off;
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                if (t < t_in) {
                    const u32x4 b = *reinterpret_cast<const u32x4*>(lds + (ok ? t * tile_bytes : 0) + off);
#pragma unroll
                    for (int f = 0; f < NOF; ++f) acc[t][f] = mfma32<F16>(a[f], b, acc[t][f]);
                }
            }
            // advance by two slots
            cg += 2;
            while (cg >= groups) {
                cg -= groups;
                if (++kw == g.KW) { kw = 0; ++kh; }
            }
        }
    }

    // ---- epilogue: bias (+ residual) + LIF over T; result row i = 8 * (r / 4) + 4 * half + r % 4 of each fragment.
    if (!pix_valid) return;
    const int64_t plane_out = static_cast<int64_t>(g.Ho) * g.Wo;
    const int64_t pix_off = static_cast<int64_t>(n) * g.Cout * plane_out + static_cast<int64_t>(oh) * g.Wo + ow;
#pragma unroll
    for (int f = 0; f < NOF; ++f) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int oc = (ocf0 + f) * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            if (oc >= g.Cout) continue;
            const int64_t o = pix_off + oc * plane_out;
            const float bv = bias[oc];
            float v = v_init != nullptr ? to_float(v_init[o]) : 0.0f;
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                if (t < g.T) {
                    float cur = (g.shared_x ? acc[0][f][r] : acc[t][f][r]) + bv;
                    if (has_residual) cur += to_float(static_cast<const XT*>(residuals.p[t])[o]);
                    spikes[t * g.spike_step_stride + o] = spike_value<XT>(lif_step(cur, v, lif));
                }
            }
            v_out[o] = from_float<VT>(v);
        }
    }
}

constexpr size_t kMaxLds = 160 * 1024;
constexpr size_t kPreferredLds = 80 * 1024;  // two workgroups per CU

// Largest number of distinct input rows (global id n * H + ih) any tile row-band touches.
int max_tile_rows(const ConvGeom& g) {
    const int total_rows = g.N * g.Ho;
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

// Chooses the output tile (TH x TW <= 128 pixels, TH rows of the flattened (n, oh) space) whose activation tile for
// `t_in` timesteps fits LDS, wasting the fewest lanes and preferring full-width rows (contiguous stores) and a
// footprint that lets two workgroups share a CU. Fills TH, TW, tiles_x, tiles_y, NR, WT. Returns the LDS bytes, 0 if
// no tile fits.
size_t plan_tile_uncached(ConvGeom& g, int t_in, bool pair_aligned) {
    const int rows = g.N * g.Ho;
    double best = -1e30;
    size_t best_bytes = 0;
    ConvGeom best_g = g;
    for (int tw = 1; tw <= g.Wo && tw <= kTilePixels; ++tw) {
        for (int px = kTilePixels; px >= 32; px >>= 1) {
            int th = px / tw;
            if (th < 1) continue;
            if (th > rows) th = rows;
            ConvGeom c = g;
            c.TW = tw;
            c.TH = th;
            c.tiles_x = (g.Wo + tw - 1) / tw;
            c.tiles_y = (rows + th - 1) / th;
            c.NR = max_tile_rows(c);
            c.WT = (tw - 1) * g.sw + g.KW + (pair_aligned ? 1 : 0);
            c.WT = (c.WT + 1) & ~1;
            const size_t bytes = static_cast<size_t>(t_in) * c.NR * c.WT * c.pitch + c.pitch;
            if (bytes > kMaxLds) continue;
            const double useful = static_cast<double>(rows) * g.Wo;
            const double issued = static_cast<double>(c.tiles_x) * c.tiles_y * kTilePixels;
            const double staged = static_cast<double>(c.NR) * c.WT / (static_cast<double>(th) * tw);
            double score = useful / issued - 0.02 * staged;
            if (tw == g.Wo) score += 0.03;
            if (bytes > kPreferredLds) score -= 0.05;
            if (score > best) { best = score; best_g = c; best_bytes = bytes; }
        }
    }
    if (best_bytes != 0) g = best_g;
    return best_bytes;
}



// Planning scans every candidate tile shape, so plans are memoised per problem geometry.
size_t plan_tile(ConvGeom& g, int t_in, bool pair_aligned) {
    using Key = std::tuple<int, int, int, int, int, int, int, int, int, int, int, int>;
    struct Plan { int TH, TW, tiles_x, tiles_y, NR, WT; size_t bytes; };
    static std::mutex mu;
    static std::map<Key, Plan> plans;
    const Key key(g.N, g.H, g.W, g.KH, g.KW, g.sh, g.sw, g.ph, g.pw, g.pitch, t_in, pair_aligned ? 1 : 0);
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = plans.find(key);
        if (it != plans.end()) {
            const Plan& p = it->second;
            g.TH = p.TH; g.TW = p.TW; g.tiles_x = p.tiles_x; g.tiles_y = p.tiles_y; g.NR = p.NR; g.WT = p.WT;
            return p.bytes;
        }
    }
    const size_t bytes = plan_tile_uncached(g, t_in, pair_aligned);
    std::lock_guard<std::mutex> lock(mu);
    plans[key] = Plan{g.TH, g.TW, g.tiles_x, g.tiles_y, g.NR, g.WT, bytes};
    return bytes;
}

template <typename XT, typename VT, int TT, int NOF>
int launch(const StepPtrs& xs, const StepPtrs& res, int has_res, ConvGeom g, const void* packed, const void* v_init,
           void* spikes, void* v_out, const LifParams& lif, hipStream_t stream) {
    g.oc_tiles = (g.Cout + 32 * NOF - 1) / (32 * NOF);
    const size_t lds = static_cast<size_t>(g.shared_x ? 1 : TT) * g.NR * g.WT * g.pitch + g.pitch;
    if (lds > kMaxLds)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: activation tile of %zu bytes exceeds LDS (W=%d, kernel %dx%d)", lds, g.W, g.KH, g.KW);
    const int64_t blocks = static_cast<int64_t>(g.tiles_x) * g.tiles_y * g.oc_tiles;
    if (blocks > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: too many tiles");
    auto kernel = conv_lif_kernel<XT, VT, TT, NOF>;
    if (lds > 64 * 1024) {
        // Opt in to the full 160 KiB of LDS once per kernel instantiation and device.
        static bool raised[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
        if (!raised[dev]) {
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
            if (err != hipSuccess) return fail(SNNF_ERR_LAUNCH, "snnf_conv_lif: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(err));
            raised[dev] = true;
        }
    }
    const PackGeom pg = make_pack_geom(g.Cout, g.Cin, g.KH, g.KW);
    const uint16_t* wp = static_cast<const uint16_t*>(packed);
    const float* bias = reinterpret_cast<const float*>(wp + packed_weight_elems(pg));
    kernel<<<dim3(static_cast<unsigned>(blocks)), kThreads, lds, stream>>>(xs, res, has_res, g, wp, bias, static_cast<const VT*>(v_init),
                                                                           static_cast<XT*>(spikes), static_cast<VT*>(v_out), lif);
    return check_launch("snnf_conv_lif");
}

template <typename XT, typename VT>
int dispatch(int tt, const StepPtrs& xs, const StepPtrs& res, int has_res, const ConvGeom& g, const void* packed,
             const void* v_init, void* spikes, void* v_out, const LifParams& lif, hipStream_t stream) {
    constexpr int NOF = 2;
    if (tt == 1) return launch<XT, VT, 1, NOF>(xs, res, has_res, g, packed, v_init, spikes, v_out, lif, stream);
    if (tt == 2) return launch<XT, VT, 2, NOF>(xs, res, has_res, g, packed, v_init, spikes, v_out, lif, stream);
    return launch<XT, VT, 4, NOF>(xs, res, has_res, g, packed, v_init, spikes, v_out, lif, stream);
}

}  // namespace
}  // namespace snnf

extern "C" size_t snnf_conv_packed_weight_bytes(int Cout, int Cin, int KH, int KW) {
    using namespace snnf;
    if (Cout < 1 || Cin < 1 || KH < 1 || KW < 1) return 0;
    const PackGeom p = make_pack_geom(Cout, Cin, KH, KW);
    return packed_weight_elems(p) * 2 + static_cast<size_t>(p.nocf) * 32 * sizeof(float);
}

extern "C" int snnf_conv_pack_weight(const void* weight, const void* bias, int w_dtype, int Cout, int Cin, int KH, int KW,
                                     int x_dtype, void* packed, size_t packed_bytes, void* stream) {
    using namespace snnf;
    if (weight == nullptr || packed == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_pack_weight: weight and packed must be non-null");
    if (Cout < 1 || Cin < 1 || KH < 1 || KW < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_pack_weight: Cout=%d Cin=%d KH=%d KW=%d", Cout, Cin, KH, KW);
    if (!valid_dtype(w_dtype) || !valid_dtype(x_dtype))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_pack_weight: unknown dtype code");
    const size_t need = snnf_conv_packed_weight_bytes(Cout, Cin, KH, KW);
    if (packed_bytes < need || !aligned_to(packed, 16))
        return fail(SNNF_ERR_WORKSPACE, "snnf_conv_pack_weight: packed buffer needs %zu bytes, 16-byte aligned", need);
    const PackGeom p = make_pack_geom(Cout, Cin, KH, KW);
    const int64_t total = static_cast<int64_t>(packed_weight_elems(p));
    uint16_t* out = static_cast<uint16_t*>(packed);
    float* bias_out = reinterpret_cast<float*>(out + total);
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    hipStream_t hs = as_stream(stream);
    const bool to_f16 = x_dtype == SNNF_F16;
#define SNNF_PACK(WT)                                                                                              \
    do {                                                                                                           \
        if (to_f16)                                                                                                \
            pack_weight_kernel<WT, true><<<dim3(blocks), 256, 0, hs>>>(static_cast<const WT*>(weight),            \
                                                                       static_cast<const WT*>(bias), p, out, bias_out); \
        else                                                                                                       \
            pack_weight_kernel<WT, false><<<dim3(blocks), 256, 0, hs>>>(static_cast<const WT*>(weight),           \
                                                                        static_cast<const WT*>(bias), p, out, bias_out); \
    } while (0)
    if (w_dtype == SNNF_F32) SNNF_PACK(float);
    else if (w_dtype == SNNF_BF16) SNNF_PACK(bf16_t);
    else SNNF_PACK(f16_t);
#undef SNNF_PACK
    return check_launch("snnf_conv_pack_weight");
}

extern "C" int snnf_conv_lif(const void* const* xs, const void* const* residuals, int T, int N, int Cin, int H, int W,
                             int x_dtype, const void* packed_weight, int Cout, int KH, int KW, int stride_h, int stride_w,
                             int pad_h, int pad_w, const void* v_init, int v_dtype, void* spikes,
                             int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset, float tau,
                             void* stream) {
    using namespace snnf;
    if (xs == nullptr || packed_weight == nullptr || spikes == nullptr || v_out == nullptr)
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
    if (static_cast<int64_t>(N) * H > 0x3fffffffLL || static_cast<int64_t>(N) * Cin * H * W > (1LL << 40))
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: input too large");

    ConvGeom g = {};
    g.N = N; g.Cin = Cin; g.H = H; g.W = W; g.Cout = Cout; g.KH = KH; g.KW = KW;
    g.sh = stride_h; g.sw = stride_w; g.ph = pad_h; g.pw = pad_w;
    g.Ho = (H + 2 * pad_h - KH) / stride_h + 1;
    g.Wo = (W + 2 * pad_w - KW) / stride_w + 1;
    const PackGeom pg = make_pack_geom(Cout, Cin, KH, KW);
    g.CK = pg.CK; g.nchunks = pg.nchunks; g.npairs = pg.npairs;
    g.groups_log2 = pg.CK == 8 ? 0 : (pg.CK == 16 ? 1 : 2);
    g.pitch = pg.CK * 2 + 16;
    const int xsize = dtype_size(x_dtype);
    g.spike_step_stride = spike_step_stride;
    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    hipStream_t hs = as_stream(stream);

    constexpr int kMaxTT = 4;
    // Timesteps per launch: as many as fit LDS side by side (a shared analog frame needs one tile for any window).
    bool all_shared = T > 1;
    bool pair_ok = xsize == 2 && (W % 2 == 0);
    for (int t = 0; t < T; ++t) {
        all_shared = all_shared && xs[t] == xs[0];
        pair_ok = pair_ok && aligned_to(xs[t], 4);
    }
    g.pair_aligned = pair_ok ? 1 : 0;
    int window = T < kMaxTT ? T : kMaxTT;
    {
        int w2 = 1;
        while (w2 < window) w2 *= 2;
        window = w2;
    }
    size_t lds_bytes = 0;
    while (true) {
        lds_bytes = plan_tile(g, all_shared ? 1 : window, pair_ok);
        if (lds_bytes != 0 || window == 1 || all_shared) break;
        window >>= 1;
    }
    if (lds_bytes == 0)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_conv_lif: no activation tile fits LDS (W=%d, kernel %dx%d, stride %dx%d)", W, KH, KW, stride_h, stride_w);

    for (int t0 = 0; t0 < T; t0 += window) {
        const int tw = (T - t0) < window ? (T - t0) : window;
        int tt = 1;
        while (tt < tw) tt *= 2;
        StepPtrs xp = {}, rp = {};
        for (int t = 0; t < tt; ++t) {
            xp.p[t] = xs[t0 + (t < tw ? t : 0)];  // padded steps repeat step 0 and are never stored
            if (residuals != nullptr) rp.p[t] = residuals[t0 + (t < tw ? t : 0)];
        }
        ConvGeom gl = g;
        gl.T = tw;
        gl.shared_x = (all_shared && tt > 1) ? 1 : 0;
        const void* vi = t0 == 0 ? v_init : v_out;
        void* sp = static_cast<char*>(spikes) + static_cast<int64_t>(t0) * spike_step_stride * xsize;
        const int has_res = residuals != nullptr ? 1 : 0;
        int rc;
        if (x_dtype == SNNF_F32) rc = dispatch<float, float>(tt, xp, rp, has_res, gl, packed_weight, vi, sp, v_out, lif, hs);
        else if (x_dtype == SNNF_BF16)
            rc = v_dtype == SNNF_F32 ? dispatch<bf16_t, float>(tt, xp, rp, has_res, gl, packed_weight, vi, sp, v_out, lif, hs)
                                     : dispatch<bf16_t, bf16_t>(tt, xp, rp, has_res, gl, packed_weight, vi, sp, v_out, lif, hs);
        else
            rc = v_dtype == SNNF_F32 ? dispatch<f16_t, float>(tt, xp, rp, has_res, gl, packed_weight, vi, sp, v_out, lif, hs)
                                     : dispatch<f16_t, f16_t>(tt, xp, rp, has_res, gl, packed_weight, vi, sp, v_out, lif, hs);
        if (rc != SNNF_OK) return rc;
    }
    return SNNF_OK;
}
