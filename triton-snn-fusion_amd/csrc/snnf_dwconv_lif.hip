// Depthwise 3x3 (padding 1, stride 1|2) + bias (+ residual) + LIF over T steps.
//
// Bound by HBM bandwidth: every activation is read once and every spike written once; the 3x3 halo re-use happens in
// LDS. A workgroup owns PB consecutive (n, c) planes (or a band of TH output rows of one plane), keeps an fp32 copy of
// the input band with a zero halo in LDS, and every thread keeps the fp32 membrane of its PX-wide output strips in
// registers for the whole time loop.
#include "snnf_common.h"

namespace snnf {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 2;     // output strips per thread
constexpr int kColOffset = 4;  // LDS column of input column 0 (keeps 16-byte alignment; column 3 is the left halo)
constexpr size_t kDwMaxLds = 64 * 1024;
typedef float dw_f32x4 __attribute__((ext_vector_type(4)));   // one 16-byte LDS access

// Input vectors a thread prefetches per timestep: a stride-2 band has about four input vectors per output strip.
template <int STRIDE>
__host__ __device__ constexpr int kLoadSlots() { return STRIDE == 1 ? 3 : 8; }

struct DwGeom {
    int planes;      // N * C
    int C, H, W, Ho, Wo;
    int TH;          // output rows per band
    int PB;          // planes per workgroup
    int bands;       // ceil(Ho / TH)
    int RIN;         // input rows held per plane: (TH - 1) * stride + 3
    int pitch;       // LDS floats per input row
    int SW;          // strips per output row = Wo / PX
    int WV;          // load vectors per input row = W / PX
};

template <typename XT, int PX>
__device__ __forceinline__ void load_strip_as_float(const XT* __restrict__ p, float (&out)[PX]) {
    const Pack<XT, PX> raw = *reinterpret_cast<const Pack<XT, PX>*>(p);
#pragma unroll
    for (int i = 0; i < PX; ++i) out[i] = to_float(raw.v[i]);
}

// Entry i of a pointer table passed by value as a kernel argument, read from the kernel-argument segment with a scalar
// load (explicit arguments start at offset 0 of that segment, in declaration order).
__device__ __forceinline__ const void* dw_table_entry(int table_offset_bytes, int i) {
    typedef const void* cvp;
    typedef const __attribute__((address_space(4))) unsigned char* ka_bytes;
    typedef const __attribute__((address_space(4))) cvp* ka_entry;
    ka_bytes ka = (ka_bytes)__builtin_amdgcn_kernarg_segment_ptr();
    return *(ka_entry)(ka + table_offset_bytes + i * 8);
}

// Pipeline of one timestep: the step's input vectors, prefetched into registers during the previous step, are widened
// to fp32 and written into one of two LDS tiles; one workgroup barrier; the previous step's spikes leave (they waited
// in registers so that the wait for the prefetched loads never finds fresh stores in front of it); the next step's
// loads are issued; then the 3x3 taps and the LIF update run on the tile. The two pointer tables MUST be the first two
// kernel parameters.
// STD: the common neuron (power-of-two tau, hard reset) inlined without per-element mode branches.
template <typename XT, typename VT, int STRIDE, int PX, bool STD>
__global__ __launch_bounds__(kThreads) void dwconv3x3_lif_kernel(StepPtrs xs, StepPtrs residuals, int has_residual,
                                                                 int T, DwGeom g, const XT* __restrict__ weight,
                                                                 const XT* __restrict__ bias,
                                                                 const VT* __restrict__ v_init,
                                                                 XT* __restrict__ spikes, int64_t spike_step_stride,
                                                                 VT* __restrict__ v_out, LifParams lif) {
    extern __shared__ __align__(16) float tile[];
    constexpr bool BITS = false;                       // dense 0 / 1 spikes only (the packed output is the dot-product kernel's)
    constexpr int IN_COLS = (PX - 1) * STRIDE + 3;
    constexpr int KL = kLoadSlots<STRIDE>();           // input vectors a thread prefetches per timestep
    constexpr uint32_t ES = static_cast<uint32_t>(sizeof(XT));

    const int tid = threadIdx.x;
    const int band = blockIdx.x % g.bands;
    const int plane0 = (blockIdx.x / g.bands) * g.PB;
    const int planes_here = min(g.PB, g.planes - plane0);
    const int row0 = band * g.TH;                       // first output row of the band
    const int rows_here = min(g.TH, g.Ho - row0);
    const int in_row0 = row0 * STRIDE - 1;              // input row held in LDS row 0
    const int plane_floats = g.RIN * g.pitch;
    const int buf_floats = g.PB * plane_floats;

    // Zero both tiles once: halo columns and out-of-image rows stay zero for every timestep.
    for (int i = tid; i < 2 * buf_floats; i += kThreads) tile[i] = 0.0f;

    // ---- fixed ownership of input vectors (PX elements of one input row) for the whole time loop.
    const int load_vectors = planes_here * g.RIN * g.WV;
    uint32_t ld_src[KL];     // byte offset from the first plane of this workgroup; 0 for an idle slot
    int ld_dst[KL];          // float offset into a tile; -1 for an idle slot
#pragma unroll
    for (int k = 0; k < KL; ++k) {
        const int i = tid + k * kThreads;
        ld_src[k] = 0;
        ld_dst[k] = -1;
        if (i < load_vectors) {
            const int p = i / (g.RIN * g.WV);
            const int rem = i - p * (g.RIN * g.WV);
            const int r = rem / g.WV;
            const int cv = rem - r * g.WV;
            const int ih = in_row0 + r;
            if (ih >= 0 && ih < g.H) {
                ld_src[k] = static_cast<uint32_t>((p * g.H + ih) * g.W + cv * PX) * ES;
                ld_dst[k] = p * plane_floats + r * g.pitch + kColOffset + cv * PX;
            }
        }
    }
    const int64_t in_base = static_cast<int64_t>(plane0) * g.H * g.W;    // elements

    // ---- fixed ownership of output strips.
    const int strips_per_plane = rows_here * g.SW;
    const int strips = planes_here * strips_per_plane;
    int item_src[kItems];          // float offset of the strip's top-left input (left halo) inside a tile
    uint32_t item_out[kItems];     // element offset of the strip from the first output plane of this workgroup
    bool item_live[kItems];
    float v[kItems][PX];
    float w[kItems][9];
    float b[kItems];
    const int64_t out_base = (static_cast<int64_t>(plane0) * g.Ho + row0) * g.Wo;   // elements
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int i = tid + k * kThreads;
        item_live[k] = i < strips;
        const int ii = item_live[k] ? i : 0;
        const int ip = ii / strips_per_plane;
        const int rem = ii - ip * strips_per_plane;
        const int ir = rem / g.SW;
        const int ic = (rem - ir * g.SW) * PX;
        item_src[k] = ip * plane_floats + (ir * STRIDE) * g.pitch + (kColOffset - 1) + ic * STRIDE;
        item_out[k] = static_cast<uint32_t>((ip * g.Ho + ir) * g.Wo + ic);
        const int c = (plane0 + ip) % g.C;
#pragma unroll
        for (int j = 0; j < 9; ++j) w[k][j] = to_float(weight[c * 9 + j]);
        b[k] = to_float(bias[c]);
        if (item_live[k] && v_init != nullptr) {
            load_strip_as_float<VT, PX>(v_init + out_base + item_out[k], v[k]);
        } else {
#pragma unroll
            for (int j = 0; j < PX; ++j) v[k][j] = 0.0f;
        }
    }

    // ---- prefetch registers and the spikes waiting to be stored.
    Pack<XT, PX> pre[KL];
    auto issue_loads = [&](int t) __attribute__((always_inline)) {
        const char* __restrict__ x = reinterpret_cast<const char*>(static_cast<const XT*>(dw_table_entry(0, t)) + in_base);
#pragma unroll
        for (int k = 0; k < KL; ++k) pre[k] = *reinterpret_cast<const Pack<XT, PX>*>(x + ld_src[k]);
    };
    Pack<XT, PX> pend[BITS ? 1 : kItems];
    uint32_t pend_bits[BITS ? kItems : 1];
    int pend_t = -1;
    auto flush = [&]() __attribute__((always_inline)) {
        if constexpr (BITS) {
            unsigned char* __restrict__ out = reinterpret_cast<unsigned char*>(spikes) + pend_t * spike_step_stride + (out_base >> 3);
#pragma unroll
            for (int k = 0; k < kItems; ++k)
                if (item_live[k]) out[item_out[k] >> 3] = static_cast<unsigned char>(pend_bits[k]);
        } else {
            XT* __restrict__ out = spikes + pend_t * spike_step_stride + out_base;
#pragma unroll
            for (int k = 0; k < kItems; ++k)
                if (item_live[k]) *reinterpret_cast<Pack<XT, PX>*>(out + item_out[k]) = pend[k];
        }
        pend_t = -1;
    };

    issue_loads(0);
    __syncthreads();   // zero fill complete
    int buf = 0;
    for (int t = 0; t < T; ++t) {
        float* __restrict__ cur = tile + buf * buf_floats;
#pragma unroll
        for (int k = 0; k < KL; ++k) {
            if (ld_dst[k] >= 0) {
                float* dst = cur + ld_dst[k];
                if constexpr (PX % 4 == 0) {
#pragma unroll
                    for (int q = 0; q < PX / 4; ++q) {
                        const dw_f32x4 four = {to_float(pre[k].v[4 * q]), to_float(pre[k].v[4 * q + 1]),
                                               to_float(pre[k].v[4 * q + 2]), to_float(pre[k].v[4 * q + 3])};
                        *reinterpret_cast<dw_f32x4*>(dst + 4 * q) = four;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < PX; ++j) dst[j] = to_float(pre[k].v[j]);
                }
            }
        }
        __syncthreads();   // tile of step t complete; every wave is past its reads of the other tile
        if (pend_t >= 0) flush();
        if (t + 1 < T) issue_loads(t + 1);

        const XT* __restrict__ res = has_residual ? static_cast<const XT*>(dw_table_entry(sizeof(StepPtrs), t)) + out_base : nullptr;
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            if (__builtin_amdgcn_ballot_w64(item_live[k]) == 0) continue;   // a wave none of whose lanes owns a strip in this round
            const float* __restrict__ src = cur + item_src[k];
            float acc[PX];
#pragma unroll
            for (int j = 0; j < PX; ++j) acc[j] = b[k];
#pragma unroll
            for (int kh = 0; kh < 3; ++kh) {
                float in[IN_COLS];
                if constexpr (PX == 8 && STRIDE == 1) {
                    // left halo, two aligned 16-byte reads, right halo
                    const float* row = src + kh * g.pitch;
                    in[0] = row[0];
                    const dw_f32x4 lo = *reinterpret_cast<const dw_f32x4*>(row + 1);
                    const dw_f32x4 hi = *reinterpret_cast<const dw_f32x4*>(row + 5);
                    in[9] = row[9];
#pragma unroll
                    for (int j = 0; j < 4; ++j) { in[1 + j] = lo[j]; in[5 + j] = hi[j]; }
                } else {
#pragma unroll
                    for (int j = 0; j < IN_COLS; ++j) in[j] = src[kh * g.pitch + j];
                }
#pragma unroll
                for (int j = 0; j < PX; ++j) {
#pragma unroll
                    for (int kw = 0; kw < 3; ++kw) acc[j] = fmaf(in[j * STRIDE + kw], w[k][kh * 3 + kw], acc[j]);
                }
            }
            if (res != nullptr && item_live[k]) {
                float r8[PX];
                load_strip_as_float<XT, PX>(res + item_out[k], r8);
#pragma unroll
                for (int j = 0; j < PX; ++j) acc[j] += r8[j];
            }
            uint32_t byte = 0;
#pragma unroll
            for (int j = 0; j < PX; ++j) {
                bool fired;
                if constexpr (STD) {
                    const float h = v[k][j] + (acc[j] - v[k][j]) * lif.inv_tau;
                    fired = h >= lif.v_threshold;
                    v[k][j] = fired ? lif.v_reset : h;
                } else {
                    fired = lif_step(acc[j], v[k][j], lif);
                }
                if constexpr (BITS) byte |= fired ? (1u << j) : 0u;
                else pend[k].v[j] = spike_value<XT>(fired);
            }
            if constexpr (BITS) pend_bits[k] = byte;
        }
        pend_t = t;
        buf ^= 1;
    }
    if (pend_t >= 0) flush();

    if (BITS && v_out == nullptr) return;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (!item_live[k]) continue;
        Pack<VT, PX> vo;
#pragma unroll
        for (int j = 0; j < PX; ++j) vo.v[j] = from_float<VT>(v[k][j]);
        *reinterpret_cast<Pack<VT, PX>*>(v_out + out_base + item_out[k]) = vo;
    }
}

template <typename XT, typename VT, int STRIDE, int PX>
int launch(const StepPtrs& xs, const StepPtrs& res, int has_res, int T, DwGeom g, const void* weight, const void* bias,
           const void* v_init, void* spikes, int64_t spike_step_stride, void* v_out, const LifParams& lif,
           hipStream_t stream) {
    g.SW = g.Wo / PX;
    g.WV = g.W / PX;
    const int max_strips = kThreads * kItems;
    const int per_plane = g.Ho * g.SW;
    if (per_plane >= max_strips) {
        g.PB = 1;
        g.TH = max_strips / g.SW;
        if (g.TH < 1) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: output row of %d pixels is too wide", g.Wo);
    } else {
        g.TH = g.Ho;
        g.PB = max_strips / per_plane;
        if (g.PB > g.planes) g.PB = g.planes;
    }
    // Row pitch: a multiple of 4 floats (16-byte vectors) but not of 8, so that the 16-byte reads of lanes that sit in
    // consecutive rows fall into different banks.
    g.pitch = ((g.W + kColOffset + 1) + 3) / 4 * 4;
    if (g.pitch % 8 == 0) g.pitch += 4;
    // Two LDS tiles (double buffering) must fit, and a thread prefetches at most kLoadSlots input vectors per timestep.
    const int max_vectors = kThreads * kLoadSlots<STRIDE>();
    auto fits = [&]() {
        g.bands = (g.Ho + g.TH - 1) / g.TH;
        g.RIN = (g.TH - 1) * STRIDE + 3;
        const size_t bytes = static_cast<size_t>(2) * g.PB * g.RIN * g.pitch * sizeof(float);
        return bytes <= kDwMaxLds && g.PB * g.RIN * g.WV <= max_vectors;
    };
    while (!fits() && g.PB > 1) g.PB = (g.PB + 1) / 2;
    while (!fits() && g.TH > 1) g.TH = (g.TH + 1) / 2;
    if (!fits()) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: input row of %d pixels does not fit LDS", g.W);
    const size_t lds = static_cast<size_t>(2) * g.PB * g.RIN * g.pitch * sizeof(float);
    const int64_t blocks = static_cast<int64_t>((g.planes + g.PB - 1) / g.PB) * g.bands;
    if (blocks > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: too many planes");
    if (lif.charge_mode == CHARGE_SCALE && !lif.soft_reset) {
        dwconv3x3_lif_kernel<XT, VT, STRIDE, PX, true><<<dim3(static_cast<unsigned>(blocks)), kThreads, lds, stream>>>(
            xs, res, has_res, T, g, static_cast<const XT*>(weight), static_cast<const XT*>(bias),
            static_cast<const VT*>(v_init), static_cast<XT*>(spikes), spike_step_stride, static_cast<VT*>(v_out), lif);
    } else {
        dwconv3x3_lif_kernel<XT, VT, STRIDE, PX, false><<<dim3(static_cast<unsigned>(blocks)), kThreads, lds, stream>>>(
            xs, res, has_res, T, g, static_cast<const XT*>(weight), static_cast<const XT*>(bias),
            static_cast<const VT*>(v_init), static_cast<XT*>(spikes), spike_step_stride, static_cast<VT*>(v_out), lif);
    }
    return check_launch("snnf_dwconv3x3_lif");
}

// ---------------------------------------------------------------------------------------------------------------
// Stride 1, strips of 8 pixels, 16-bit activations: the LDS tile keeps the activations in their 16-bit form (a prefetched
// vector goes in with one 16-byte write and no conversion) and the taps run on the packed dot-product instruction
// (two 16-bit products added to an fp32 accumulator): the products are exact in fp32, as with an fp32 multiply-add, and an
// output takes two instructions per kernel row instead of three. This kernel is bound by its vector and LDS instructions
// (with a third of the taps it runs at 6.5 TB/s), so the count is what matters.
// Row layout: input column c at element kDotColOffset + c; the elements before and after the row are the zero halo. For
// the strip at elements e0 .. e0 + 7 (e0 a multiple of 8) a row costs one 16-byte read and the two dwords around it.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kDotColOffset = 8;
typedef uint32_t dw_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 dw_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 dw_f16x2 __attribute__((ext_vector_type(2)));

template <typename XT>
__device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float c) {
    if constexpr (dtype_of<XT>::value == SNNF_BF16)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(dw_bf16x2, a), __builtin_bit_cast(dw_bf16x2, b), c, false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_f16x2, a), __builtin_bit_cast(dw_f16x2, b), c, false);
}

// BITS: the spikes of a strip and timestep leave as one byte (bit j = pixel 8 x + j of the row) instead of eight 16-bit
// values: [T][N][C][Ho][Wo / 8] bytes, `spike_step_stride` then counts bytes; the final membrane is optional.
// BITS_IN: the input spikes arrive row-packed as well ([N][C][H][W / 8] bytes per timestep): a thread fetches one byte where it
// fetched a 16-byte vector and expands it on its way into LDS.
template <typename XT, typename VT, bool STD, bool BITS = false, bool BITS_IN = false>
__global__ __launch_bounds__(kThreads) void dwconv3x3_lif_dot_kernel(StepPtrs xs, StepPtrs residuals, int has_residual,
                                                                     int T, DwGeom g, const XT* __restrict__ weight,
                                                                     const XT* __restrict__ bias,
                                                                     const VT* __restrict__ v_init,
                                                                     XT* __restrict__ spikes, int64_t spike_step_stride,
                                                                     VT* __restrict__ v_out, LifParams lif) {
    extern __shared__ __align__(16) unsigned char dot_tile_bytes[];
    uint16_t* __restrict__ tile = reinterpret_cast<uint16_t*>(dot_tile_bytes);
    constexpr int PX = 8;
    constexpr int KL = kLoadSlots<1>();
    constexpr uint32_t ES = 2;
    static_assert(sizeof(XT) == 2, "16-bit activations only");

    const int tid = threadIdx.x;
    const int band = blockIdx.x % g.bands;
    const int plane0 = (blockIdx.x / g.bands) * g.PB;
    const int planes_here = min(g.PB, g.planes - plane0);
    const int row0 = band * g.TH;
    const int rows_here = min(g.TH, g.Ho - row0);
    const int in_row0 = row0 - 1;                      // input row held in LDS row 0
    const int plane_elems = g.RIN * g.pitch;           // pitch: 16-bit elements per LDS row, a multiple of 8
    const int buf_elems = g.PB * plane_elems;

    // Zero both tiles once: halo columns and out-of-image rows stay zero for every timestep.
    for (int i = tid; i < buf_elems; i += kThreads) reinterpret_cast<uint32_t*>(tile)[i] = 0u;   // 2 tiles x buf_elems / 2 dwords

    // ---- fixed ownership of input vectors (8 elements of one input row) for the whole time loop.
    const int load_vectors = planes_here * g.RIN * g.WV;
    uint32_t ld_src[KL];     // byte offset from the first plane of this workgroup; 0 for an idle slot
    int ld_dst[KL];          // element offset into a tile; -1 for an idle slot
#pragma unroll
    for (int k = 0; k < KL; ++k) {
        const int i = tid + k * kThreads;
        ld_src[k] = 0;
        ld_dst[k] = -1;
        if (i < load_vectors) {
            const int p = i / (g.RIN * g.WV);
            const int rem = i - p * (g.RIN * g.WV);
            const int r = rem / g.WV;
            const int cv = rem - r * g.WV;
            const int ih = in_row0 + r;
            if (ih >= 0 && ih < g.H) {
                ld_src[k] = BITS_IN ? static_cast<uint32_t>((p * g.H + ih) * g.WV + cv)      // bytes: one per 8 pixels
                                    : static_cast<uint32_t>((p * g.H + ih) * g.W + cv * PX) * ES;
                ld_dst[k] = p * plane_elems + r * g.pitch + kDotColOffset + cv * PX;
            }
        }
    }
    const int64_t in_base = static_cast<int64_t>(plane0) * g.H * g.W;    // elements

    // ---- fixed ownership of output strips; the weights of a strip's channel as the four operand pairs of a kernel row:
    // (w1, w2) and (0, w0) serve the even outputs, (w0, w1) and (w2, 0) the odd ones.
    const int strips_per_plane = rows_here * g.SW;
    const int strips = planes_here * strips_per_plane;
    int item_src[kItems];          // element offset of the strip's first input pixel inside a tile (a multiple of 8)
    uint32_t item_out[kItems];     // element offset of the strip from the first output plane of this workgroup
    bool item_live[kItems];
    float v[kItems][PX];
    uint32_t wp[kItems][3][4];
    float b[kItems];
    const int64_t out_base = (static_cast<int64_t>(plane0) * g.Ho + row0) * g.Wo;   // elements
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int i = tid + k * kThreads;
        item_live[k] = i < strips;
        const int ii = item_live[k] ? i : 0;
        const int ip = ii / strips_per_plane;
        const int rem = ii - ip * strips_per_plane;
        const int ir = rem / g.SW;
        const int ic = (rem - ir * g.SW) * PX;
        item_src[k] = ip * plane_elems + ir * g.pitch + kDotColOffset + ic;
        item_out[k] = static_cast<uint32_t>((ip * g.Ho + ir) * g.Wo + ic);
        const int c = (plane0 + ip) % g.C;
        const uint16_t* __restrict__ wbits = reinterpret_cast<const uint16_t*>(weight) + c * 9;
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
            const uint32_t w0 = wbits[kh * 3], w1 = wbits[kh * 3 + 1], w2 = wbits[kh * 3 + 2];
            wp[k][kh][0] = w1 | (w2 << 16);
            wp[k][kh][1] = w0 << 16;
            wp[k][kh][2] = w0 | (w1 << 16);
            wp[k][kh][3] = w2;
        }
        b[k] = to_float(bias[c]);
        if (item_live[k] && v_init != nullptr) {
            load_strip_as_float<VT, PX>(v_init + out_base + item_out[k], v[k]);
        } else {
#pragma unroll
            for (int j = 0; j < PX; ++j) v[k][j] = 0.0f;
        }
    }

    // ---- prefetch registers and the spikes waiting to be stored.
    dw_u32x4 pre[BITS_IN ? 1 : KL];
    uint32_t pre_byte[BITS_IN ? KL : 1];
    auto issue_loads = [&](int t) __attribute__((always_inline)) {
        if constexpr (BITS_IN) {
            const unsigned char* __restrict__ x = static_cast<const unsigned char*>(dw_table_entry(0, t)) + (in_base >> 3);
#pragma unroll
            for (int k = 0; k < KL; ++k) pre_byte[k] = x[ld_src[k]];
        } else {
            const char* __restrict__ x = reinterpret_cast<const char*>(static_cast<const XT*>(dw_table_entry(0, t)) + in_base);
#pragma unroll
            for (int k = 0; k < KL; ++k) pre[k] = *reinterpret_cast<const dw_u32x4*>(x + ld_src[k]);
        }
    };
    // Eight spike bits -> eight 16-bit ones or zeros (pixel j in element j).
    auto expand = [&](uint32_t byte) __attribute__((always_inline)) -> dw_u32x4 {
        constexpr uint32_t ONE = dtype_of<XT>::value == SNNF_F16 ? 0x3c00u : 0x3f80u;
        const uint32_t m = __umul24(byte, 0x8001u);   // bit i of the byte at bits i and 15 + i
        dw_u32x4 d;
        d[0] = __umul24(m & 0x10001u, ONE);
        d[1] = __umul24((m >> 2) & 0x10001u, ONE);
        d[2] = __umul24((m >> 4) & 0x10001u, ONE);
        d[3] = __umul24((m >> 6) & 0x10001u, ONE);
        return d;
    };
    Pack<XT, PX> pend[BITS ? 1 : kItems];
    uint32_t pend_bits[BITS ? kItems : 1];
    int pend_t = -1;
    auto flush = [&]() __attribute__((always_inline)) {
        if constexpr (BITS) {
            unsigned char* __restrict__ out = reinterpret_cast<unsigned char*>(spikes) + pend_t * spike_step_stride + (out_base >> 3);
#pragma unroll
            for (int k = 0; k < kItems; ++k)
                if (item_live[k]) out[item_out[k] >> 3] = static_cast<unsigned char>(pend_bits[k]);
        } else {
            XT* __restrict__ out = spikes + pend_t * spike_step_stride + out_base;
#pragma unroll
            for (int k = 0; k < kItems; ++k)
                if (item_live[k]) *reinterpret_cast<Pack<XT, PX>*>(out + item_out[k]) = pend[k];
        }
        pend_t = -1;
    };

    issue_loads(0);
    __syncthreads();   // zero fill complete
    int buf = 0;
    for (int t = 0; t < T; ++t) {
        uint16_t* __restrict__ cur = tile + buf * buf_elems;
#pragma unroll
        for (int k = 0; k < KL; ++k) {
            if constexpr (BITS_IN) {
                if (ld_dst[k] >= 0) *reinterpret_cast<dw_u32x4*>(cur + ld_dst[k]) = expand(pre_byte[k]);
            } else {
                if (ld_dst[k] >= 0) *reinterpret_cast<dw_u32x4*>(cur + ld_dst[k]) = pre[k];
            }
        }
        __syncthreads();   // tile of step t complete; every wave is past its reads of the other tile
        if (pend_t >= 0) flush();
        if (t + 1 < T) issue_loads(t + 1);

        const XT* __restrict__ res = has_residual ? static_cast<const XT*>(dw_table_entry(sizeof(StepPtrs), t)) + out_base : nullptr;
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            if (__builtin_amdgcn_ballot_w64(item_live[k]) == 0) continue;   // a wave none of whose lanes owns a strip in this round
            const uint16_t* __restrict__ src = cur + item_src[k];
            float acc[PX];
#pragma unroll
            for (int j = 0; j < PX; ++j) acc[j] = b[k];
#pragma unroll
            for (int kh = 0; kh < 3; ++kh) {
                const uint16_t* __restrict__ row = src + kh * g.pitch;
                const dw_u32x4 d = *reinterpret_cast<const dw_u32x4*>(row);
                const uint32_t left = *reinterpret_cast<const uint32_t*>(row - 2);     // (x[-2], x[-1])
                const uint32_t right = *reinterpret_cast<const uint32_t*>(row + 8);    // (x[8], x[9])
                const uint32_t A = wp[k][kh][0], B = wp[k][kh][1], C = wp[k][kh][2], D = wp[k][kh][3];
                acc[0] = dot2_acc<XT>(d[0], A, dot2_acc<XT>(left, B, acc[0]));
                acc[1] = dot2_acc<XT>(d[0], C, dot2_acc<XT>(d[1], D, acc[1]));
                acc[2] = dot2_acc<XT>(d[1], A, dot2_acc<XT>(d[0], B, acc[2]));
                acc[3] = dot2_acc<XT>(d[1], C, dot2_acc<XT>(d[2], D, acc[3]));
                acc[4] = dot2_acc<XT>(d[2], A, dot2_acc<XT>(d[1], B, acc[4]));
                acc[5] = dot2_acc<XT>(d[2], C, dot2_acc<XT>(d[3], D, acc[5]));
                acc[6] = dot2_acc<XT>(d[3], A, dot2_acc<XT>(d[2], B, acc[6]));
                acc[7] = dot2_acc<XT>(d[3], C, dot2_acc<XT>(right, D, acc[7]));
            }
            if (res != nullptr && item_live[k]) {
                float r8[PX];
                load_strip_as_float<XT, PX>(res + item_out[k], r8);
#pragma unroll
                for (int j = 0; j < PX; ++j) acc[j] += r8[j];
            }
            uint32_t byte = 0;
#pragma unroll
            for (int j = 0; j < PX; ++j) {
                bool fired;
                if constexpr (STD) {
                    const float h = v[k][j] + (acc[j] - v[k][j]) * lif.inv_tau;
                    fired = h >= lif.v_threshold;
                    v[k][j] = fired ? lif.v_reset : h;
                } else {
                    fired = lif_step(acc[j], v[k][j], lif);
                }
                if constexpr (BITS) byte |= fired ? (1u << j) : 0u;
                else pend[k].v[j] = spike_value<XT>(fired);
            }
            if constexpr (BITS) pend_bits[k] = byte;
        }
        pend_t = t;
        buf ^= 1;
    }
    if (pend_t >= 0) flush();

    if (BITS && v_out == nullptr) return;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (!item_live[k]) continue;
        Pack<VT, PX> vo;
#pragma unroll
        for (int j = 0; j < PX; ++j) vo.v[j] = from_float<VT>(v[k][j]);
        *reinterpret_cast<Pack<VT, PX>*>(v_out + out_base + item_out[k]) = vo;
    }
}

// Launcher of the packed dot-product kernel: the planning of `launch` with 16-bit rows.
template <typename XT, typename VT, bool BITS = false, bool BITS_IN = false>
int launch_dot(const StepPtrs& xs, const StepPtrs& res, int has_res, int T, DwGeom g, const void* weight, const void* bias,
               const void* v_init, void* spikes, int64_t spike_step_stride, void* v_out, const LifParams& lif,
               hipStream_t stream) {
    constexpr int PX = 8;
    g.SW = g.Wo / PX;
    g.WV = g.W / PX;
    const int max_strips = kThreads * kItems;
    const int per_plane = g.Ho * g.SW;
    if (per_plane >= max_strips) {
        g.PB = 1;
        g.TH = max_strips / g.SW;
        if (g.TH < 1) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: output row of %d pixels is too wide", g.Wo);
    } else {
        g.TH = g.Ho;
        g.PB = max_strips / per_plane;
        if (g.PB > g.planes) g.PB = g.planes;
    }
    // Row pitch in 16-bit elements: the row, its offset and two halo elements behind it, rounded to 16 bytes; not a multiple
    // of 128 bytes, so that the 16-byte reads of lanes that sit in consecutive rows fall into different banks.
    g.pitch = (g.W + kDotColOffset + 2 + 7) / 8 * 8;
    if (g.pitch % 64 == 0) g.pitch += 8;
    const int max_vectors = kThreads * kLoadSlots<1>();
    auto fits = [&]() {
        g.bands = (g.Ho + g.TH - 1) / g.TH;
        g.RIN = g.TH + 2;
        const size_t bytes = static_cast<size_t>(2) * g.PB * g.RIN * g.pitch * sizeof(uint16_t);
        return bytes <= kDwMaxLds && g.PB * g.RIN * g.WV <= max_vectors;
    };
    while (!fits() && g.PB > 1) g.PB = (g.PB + 1) / 2;
    while (!fits() && g.TH > 1) g.TH = (g.TH + 1) / 2;
    if (!fits()) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: input row of %d pixels does not fit LDS", g.W);
    const size_t lds = static_cast<size_t>(2) * g.PB * g.RIN * g.pitch * sizeof(uint16_t);
    const int64_t blocks = static_cast<int64_t>((g.planes + g.PB - 1) / g.PB) * g.bands;
    if (blocks > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: too many planes");
    if (lif.charge_mode == CHARGE_SCALE && !lif.soft_reset) {
        dwconv3x3_lif_dot_kernel<XT, VT, true, BITS, BITS_IN><<<dim3(static_cast<unsigned>(blocks)), kThreads, lds, stream>>>(
            xs, res, has_res, T, g, static_cast<const XT*>(weight), static_cast<const XT*>(bias),
            static_cast<const VT*>(v_init), static_cast<XT*>(spikes), spike_step_stride, static_cast<VT*>(v_out), lif);
    } else {
        dwconv3x3_lif_dot_kernel<XT, VT, false, BITS, BITS_IN><<<dim3(static_cast<unsigned>(blocks)), kThreads, lds, stream>>>(
            xs, res, has_res, T, g, static_cast<const XT*>(weight), static_cast<const XT*>(bias),
            static_cast<const VT*>(v_init), static_cast<XT*>(spikes), spike_step_stride, static_cast<VT*>(v_out), lif);
    }
    return check_launch("snnf_dwconv3x3_lif");
}


template <typename XT, typename VT, int STRIDE>
int dispatch_px(int px, const StepPtrs& xs, const StepPtrs& res, int has_res, int T, const DwGeom& g,
                const void* weight, const void* bias, const void* v_init, void* spikes, int64_t sss, void* v_out,
                const LifParams& lif, hipStream_t stream) {
    if constexpr (STRIDE == 1 && sizeof(XT) == 2) {
        if (px == 8) return launch_dot<XT, VT>(xs, res, has_res, T, g, weight, bias, v_init, spikes, sss, v_out, lif, stream);
    }
    if (px == 8) return launch<XT, VT, STRIDE, 8>(xs, res, has_res, T, g, weight, bias, v_init, spikes, sss, v_out, lif, stream);
    if (px == 4) return launch<XT, VT, STRIDE, 4>(xs, res, has_res, T, g, weight, bias, v_init, spikes, sss, v_out, lif, stream);
    return launch<XT, VT, STRIDE, 1>(xs, res, has_res, T, g, weight, bias, v_init, spikes, sss, v_out, lif, stream);
}

template <typename XT, typename VT>
int dispatch_stride(int stride, int px, const StepPtrs& xs, const StepPtrs& res, int has_res, int T, const DwGeom& g,
                    const void* weight, const void* bias, const void* v_init, void* spikes, int64_t sss, void* v_out,
                    const LifParams& lif, hipStream_t stream) {
    if (stride == 1) return dispatch_px<XT, VT, 1>(px, xs, res, has_res, T, g, weight, bias, v_init, spikes, sss, v_out, lif, stream);
    return dispatch_px<XT, VT, 2>(px, xs, res, has_res, T, g, weight, bias, v_init, spikes, sss, v_out, lif, stream);
}

// One byte of row-packed spikes -> eight 0 / 1 elements (16 bytes).
template <typename XT>
__global__ __launch_bounds__(kThreads) void rowbits_unpack_kernel(const unsigned char* __restrict__ bits, XT* __restrict__ dense, int64_t bytes) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= bytes) return;
    const uint32_t b = bits[i];
    Pack<XT, 8> out;
#pragma unroll
    for (int j = 0; j < 8; ++j) out.v[j] = spike_value<XT>(((b >> j) & 1u) != 0u);
    *reinterpret_cast<Pack<XT, 8>*>(dense + i * 8) = out;
}

// Eight dense elements (16 bytes) -> one byte of row-packed spikes (bit j = element j != 0).
template <typename XT>
__global__ __launch_bounds__(kThreads) void rowbits_pack_kernel(const XT* __restrict__ dense, unsigned char* __restrict__ bits, int64_t bytes) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= bytes) return;
    const Pack<XT, 8> in = *reinterpret_cast<const Pack<XT, 8>*>(dense + i * 8);
    uint32_t b = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) b |= to_float(in.v[j]) != 0.0f ? (1u << j) : 0u;
    bits[i] = static_cast<unsigned char>(b);
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_rowbits_pack(const void* dense, void* bits, int64_t bytes, int x_dtype, void* stream) {
    using namespace snnf;
    if (bits == nullptr || dense == nullptr || bytes < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_rowbits_pack: dense and bits must be non-null, bytes >= 1");
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_rowbits_pack: unsupported_dtype: bf16 or fp16");
    if (!aligned_to(dense, 16)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_rowbits_pack: dense must be 16-byte aligned");
    const int64_t blocks = (bytes + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_rowbits_pack: too many bytes");
    hipStream_t hs = as_stream(stream);
    if (x_dtype == SNNF_BF16)
        rowbits_pack_kernel<bf16_t><<<dim3(static_cast<unsigned>(blocks)), kThreads, 0, hs>>>(static_cast<const bf16_t*>(dense), static_cast<unsigned char*>(bits), bytes);
    else
        rowbits_pack_kernel<f16_t><<<dim3(static_cast<unsigned>(blocks)), kThreads, 0, hs>>>(static_cast<const f16_t*>(dense), static_cast<unsigned char*>(bits), bytes);
    return check_launch("snnf_rowbits_pack");
}

extern "C" int snnf_dwconv3x3_lif_rowbits(const void* const* xs, const void* const* residuals, int T, int N, int C, int H, int W,
                                          int x_dtype, int x_packed, const void* weight, const void* bias, const void* v_init,
                                          void* spike_bits, int64_t bits_step_stride, void* v_out,
                                          float v_threshold, float v_reset, float tau, void* stream) {
    using namespace snnf;
    const char* who = "snnf_dwconv3x3_lif_rowbits";
    if (xs == nullptr || weight == nullptr || bias == nullptr || spike_bits == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: xs, weight, bias and spike_bits must be non-null", who);
    if (T < 1 || N < 1 || C < 1 || H < 1 || W < 1) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: T=%d N=%d C=%d H=%d W=%d", who, T, N, C, H, W);
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_dtype: activations must be bf16 or fp16", who);
    if (W % 8 != 0) return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: W=%d is not a multiple of 8", who, W);
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_tau: tau must be nonzero", who);
    if (static_cast<int64_t>(N) * C > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "%s: N*C too large", who);
    if (v_out == nullptr && T > SNNF_MAX_T_PER_LAUNCH)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: v_out is required beyond %d timesteps (the membrane passes from launch to launch)", who,
                    SNNF_MAX_T_PER_LAUNCH);
    const int64_t frame_bytes = static_cast<int64_t>(N) * C * H * (W / 8);
    if (bits_step_stride < frame_bytes) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: bits_step_stride=%lld is less than one timestep (%lld bytes)", who,
                                                    (long long)bits_step_stride, (long long)frame_bytes);
    bool aligned = (v_init == nullptr || aligned_to(v_init, 16)) && (v_out == nullptr || aligned_to(v_out, 16));
    for (int t = 0; t < T; ++t) {
        if (xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: xs[%d] is null", who, t);
        if (residuals != nullptr && residuals[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: residuals[%d] is null", who, t);
        aligned = aligned && (x_packed != 0 || aligned_to(xs[t], 16)) && (residuals == nullptr || aligned_to(residuals[t], 16));
    }
    if (!aligned) return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_alignment: activations, residuals and membranes must be 16-byte aligned", who);

    DwGeom g = {};
    g.planes = N * C;
    g.C = C;
    g.H = H;
    g.W = W;
    g.Ho = H;
    g.Wo = W;
    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    hipStream_t hs = as_stream(stream);
    for (int t0 = 0; t0 < T; t0 += SNNF_MAX_T_PER_LAUNCH) {
        const int tw = (T - t0) < SNNF_MAX_T_PER_LAUNCH ? (T - t0) : SNNF_MAX_T_PER_LAUNCH;
        StepPtrs xp = {}, rp = {};
        for (int t = 0; t < tw; ++t) {
            xp.p[t] = xs[t0 + t];
            if (residuals != nullptr) rp.p[t] = residuals[t0 + t];
        }
        const void* vi = t0 == 0 ? v_init : v_out;
        void* sp = static_cast<char*>(spike_bits) + static_cast<int64_t>(t0) * bits_step_stride;
        const int has_res = residuals != nullptr ? 1 : 0;
        int rc;
        if (x_packed != 0)
            rc = x_dtype == SNNF_BF16
                     ? launch_dot<bf16_t, float, true, true>(xp, rp, has_res, tw, g, weight, bias, vi, sp, bits_step_stride, v_out, lif, hs)
                     : launch_dot<f16_t, float, true, true>(xp, rp, has_res, tw, g, weight, bias, vi, sp, bits_step_stride, v_out, lif, hs);
        else
            rc = x_dtype == SNNF_BF16
                     ? launch_dot<bf16_t, float, true>(xp, rp, has_res, tw, g, weight, bias, vi, sp, bits_step_stride, v_out, lif, hs)
                     : launch_dot<f16_t, float, true>(xp, rp, has_res, tw, g, weight, bias, vi, sp, bits_step_stride, v_out, lif, hs);
        if (rc != SNNF_OK) return rc;
    }
    return SNNF_OK;
}

extern "C" int snnf_rowbits_unpack(const void* bits, void* dense, int64_t bytes, int x_dtype, void* stream) {
    using namespace snnf;
    if (bits == nullptr || dense == nullptr || bytes < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_rowbits_unpack: bits and dense must be non-null, bytes >= 1");
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_rowbits_unpack: unsupported_dtype: bf16 or fp16");
    if (!aligned_to(dense, 16)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_rowbits_unpack: dense must be 16-byte aligned");
    const int64_t blocks = (bytes + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_rowbits_unpack: too many bytes");
    hipStream_t hs = as_stream(stream);
    if (x_dtype == SNNF_BF16)
        rowbits_unpack_kernel<bf16_t><<<dim3(static_cast<unsigned>(blocks)), kThreads, 0, hs>>>(static_cast<const unsigned char*>(bits), static_cast<bf16_t*>(dense), bytes);
    else
        rowbits_unpack_kernel<f16_t><<<dim3(static_cast<unsigned>(blocks)), kThreads, 0, hs>>>(static_cast<const unsigned char*>(bits), static_cast<f16_t*>(dense), bytes);
    return check_launch("snnf_rowbits_unpack");
}

extern "C" int snnf_dwconv3x3_lif(const void* const* xs, const void* const* residuals, int T, int N, int C, int H, int W,
                                  int stride, int x_dtype, const void* weight, const void* bias, int w_dtype,
                                  const void* v_init, int v_dtype, void* spikes, int64_t spike_step_stride, void* v_out,
                                  float v_threshold, float v_reset, float tau, void* stream) {
    using namespace snnf;
    if (xs == nullptr || weight == nullptr || bias == nullptr || spikes == nullptr || v_out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_dwconv3x3_lif: xs, weight, bias, spikes and v_out must be non-null");
    if (T < 1 || N < 1 || C < 1 || H < 1 || W < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_dwconv3x3_lif: T=%d N=%d C=%d H=%d W=%d", T, N, C, H, W);
    if (stride != 1 && stride != 2)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: unsupported_stride: 3x3 depthwise supports stride 1 or 2, got %d", stride);
    if (!valid_dtype(x_dtype) || !valid_dtype(v_dtype) || !valid_dtype(w_dtype))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_dwconv3x3_lif: unknown dtype code");
    if (w_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: unsupported_dtype: weight/bias dtype must match x");
    if (v_dtype != SNNF_F32 && v_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: unsupported_dtype: membrane dtype must be fp32 or the activation dtype");
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: unsupported_tau: tau must be nonzero");
    if (static_cast<int64_t>(N) * C > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_dwconv3x3_lif: N*C too large");
    for (int t = 0; t < T; ++t) {
        if (xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_dwconv3x3_lif: xs[%d] is null", t);
        if (residuals != nullptr && residuals[t] == nullptr)
            return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_dwconv3x3_lif: residuals[%d] is null", t);
    }

    DwGeom g = {};
    g.planes = N * C;
    g.C = C;
    g.H = H;
    g.W = W;
    g.Ho = (H + 2 - 3) / stride + 1;
    g.Wo = (W + 2 - 3) / stride + 1;
    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    const int xsize = dtype_size(x_dtype);
    const int vsize = dtype_size(v_dtype);
    hipStream_t hs = as_stream(stream);

    for (int t0 = 0; t0 < T; t0 += SNNF_MAX_T_PER_LAUNCH) {
        const int tw = (T - t0) < SNNF_MAX_T_PER_LAUNCH ? (T - t0) : SNNF_MAX_T_PER_LAUNCH;
        StepPtrs xp = {}, rp = {};
        const void* vi = t0 == 0 ? v_init : v_out;
        void* sp = static_cast<char*>(spikes) + static_cast<int64_t>(t0) * spike_step_stride * xsize;
        // Widest strip for which every row start of every operand is naturally aligned.
        int px = 1;
        for (int cand : {8, 4}) {
            const size_t xa = static_cast<size_t>(cand) * xsize;
            const size_t va = static_cast<size_t>(cand) * vsize > 16 ? 16 : static_cast<size_t>(cand) * vsize;
            bool ok = g.Wo % cand == 0 && g.W % cand == 0 && spike_step_stride % cand == 0 && aligned_to(sp, xa) &&
                      aligned_to(v_out, va) && (vi == nullptr || aligned_to(vi, va));
            for (int t = 0; t < tw && ok; ++t) {
                ok = aligned_to(xs[t0 + t], xa);
                if (residuals != nullptr) ok = ok && aligned_to(residuals[t0 + t], xa);
            }
            if (ok) { px = cand; break; }
        }
        for (int t = 0; t < tw; ++t) {
            xp.p[t] = xs[t0 + t];
            if (residuals != nullptr) rp.p[t] = residuals[t0 + t];
        }
        const int has_res = residuals != nullptr ? 1 : 0;
        int rc;
        if (x_dtype == SNNF_F32) {
            rc = dispatch_stride<float, float>(stride, px, xp, rp, has_res, tw, g, weight, bias, vi, sp, spike_step_stride, v_out, lif, hs);
        } else if (x_dtype == SNNF_BF16) {
            rc = v_dtype == SNNF_F32
                     ? dispatch_stride<bf16_t, float>(stride, px, xp, rp, has_res, tw, g, weight, bias, vi, sp, spike_step_stride, v_out, lif, hs)
                     : dispatch_stride<bf16_t, bf16_t>(stride, px, xp, rp, has_res, tw, g, weight, bias, vi, sp, spike_step_stride, v_out, lif, hs);
        } else {
            rc = v_dtype == SNNF_F32
                     ? dispatch_stride<f16_t, float>(stride, px, xp, rp, has_res, tw, g, weight, bias, vi, sp, spike_step_stride, v_out, lif, hs)
                     : dispatch_stride<f16_t, f16_t>(stride, px, xp, rp, has_res, tw, g, weight, bias, vi, sp, spike_step_stride, v_out, lif, hs);
        }
        if (rc != SNNF_OK) return rc;
    }
    return SNNF_OK;
}
