// Temporal Linear + LIF on the matrix cores: out^T[Fout, T*M] = W[Fout, Fin] . x^T, LIF recurrence in the epilogue.
//
// Both operands are K-contiguous in memory (x rows and W rows), which is the per-lane operand order of
// v_mfma_f32_16x16x32 (8 consecutive k per lane). All T timesteps of a row tile share one weight fragment (the weight is
// streamed once per workgroup, not once per timestep), and each thread runs the LIF recurrence over T for its (row,
// output feature) pair with the membrane in a register. Two kernels: the staged one (4 timesteps or more, aligned rows)
// moves K slabs of all operand rows through LDS with coalesced loads; the direct one (everything else) loads fragments
// straight from global memory, its 8 (beyond 8 timesteps, 4) waves splitting K in pairs of K steps with partial sums
// meeting in LDS.
#include <algorithm>

#include "snnf_common.h"

namespace snnf {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileOC = 16;   // output features per workgroup
constexpr int kTileM = 16;    // rows per workgroup (per timestep)

// fp32 tensors: both operands enter the matrix cores as two bf16 terms (value rounded to bf16, and the rounded remainder),
// and three of the four products are accumulated: w_hi x_hi + w_lo x_hi + w_hi x_lo (the fourth is below 2^-16 of the
// result). The three products are three passes over K ("K parts"): part 0 multiplies the high terms, part 1 the weights' low
// terms with the activations' high terms, part 2 the other way round. 16-bit tensors have one part.
struct LinGeom {
    int T, M, Fin, Fout;
    int64_t x_row_stride;      // elements
    int64_t spike_step_stride; // elements
    int ksteps;                // ceil(Fin / 32)
    int kparts;                // 1, or 3 for fp32 tensors
};

// Eight consecutive K elements of one row as a matrix-core operand (bf16 for fp32/bf16 storage, fp16 for fp16 storage).
template <typename XT> struct Frag;
template <> struct Frag<bf16_t> { using type = bf16x8; };
template <> struct Frag<float> { using type = bf16x8; };
template <> struct Frag<f16_t> { using type = f16x8; };

// Two fp32 values as a pair of bf16 terms: their roundings to bf16, or (low_term) what those roundings left over.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi, bool low_term) {
    return split_bf16_bits(lo, low_term) | (split_bf16_bits(hi, low_term) << 16);
}

// Loads k .. k+7 of `row`; elements at or beyond `kmax` read as zero. FAST requires 16-byte aligned rows and kmax % 8 == 0
// and is branch-free (an octet beyond kmax re-reads the row's first one and is zeroed): a branch around a load would make
// the compiler wait for every load before it issues the next.
template <typename XT, bool FAST>
__device__ __forceinline__ u32x4 load_octet(const XT* __restrict__ row, int k, int kmax, bool low_term = false) {
    u32x4 out = {0u, 0u, 0u, 0u};
    if constexpr (FAST) {
        const bool inside = k < kmax;
        const XT* __restrict__ src = row + (inside ? k : 0);
        if constexpr (sizeof(XT) == 2) {
            out = *reinterpret_cast<const u32x4*>(src);
        } else {
            const f32x4 a = *reinterpret_cast<const f32x4*>(src);
            const f32x4 b = *reinterpret_cast<const f32x4*>(src + 4);
            out[0] = pack_bf16x2(a[0], a[1], low_term);
            out[1] = pack_bf16x2(a[2], a[3], low_term);
            out[2] = pack_bf16x2(b[0], b[1], low_term);
            out[3] = pack_bf16x2(b[2], b[3], low_term);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) out[j] = inside ? out[j] : 0u;
    } else if constexpr (sizeof(XT) == 2) {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(row);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = (k + 2 * j) < kmax ? p[k + 2 * j] : 0u;
            const uint32_t hi = (k + 2 * j + 1) < kmax ? p[k + 2 * j + 1] : 0u;
            out[j] = lo | (hi << 16);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float lo = (k + 2 * j) < kmax ? to_float(row[k + 2 * j]) : 0.0f;
            const float hi = (k + 2 * j + 1) < kmax ? to_float(row[k + 2 * j + 1]) : 0.0f;
            out[j] = pack_bf16x2(lo, hi, low_term);
        }
    }
    return out;
}

// The same octet in two steps, for loads that stay in flight over other work: the raw 16 (fp32 storage: 32) bytes as
// loaded, and their conversion to a matrix operand (zero when the octet lies beyond K) at the point of use. Converting
// where the load is issued would make the wave wait for it there.
template <typename XT> struct RawOctet { u32x4 lo; };
template <> struct RawOctet<float> { f32x4 lo, hi; };
template <typename XT>
__device__ __forceinline__ RawOctet<XT> load_raw_octet(const XT* __restrict__ src) {
    RawOctet<XT> r;
    if constexpr (sizeof(XT) == 2) {
        r.lo = *reinterpret_cast<const u32x4*>(src);
    } else {
        r.lo = *reinterpret_cast<const f32x4*>(src);
        r.hi = *reinterpret_cast<const f32x4*>(src + 4);
    }
    return r;
}
template <typename XT>
__device__ __forceinline__ u32x4 finish_octet(const RawOctet<XT>& r, bool inside, bool low_term) {
    u32x4 out;
    if constexpr (sizeof(XT) == 2) {
        out = r.lo;
    } else {
        out[0] = pack_bf16x2(r.lo[0], r.lo[1], low_term);
        out[1] = pack_bf16x2(r.lo[2], r.lo[3], low_term);
        out[2] = pack_bf16x2(r.hi[0], r.hi[1], low_term);
        out[3] = pack_bf16x2(r.hi[2], r.hi[3], low_term);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = inside ? out[j] : 0u;
    return out;
}

// Eight features at one bit each (bit j = feature j) as a matrix operand of zeros and ones.
template <typename XT>
__device__ __forceinline__ u32x4 expand_bit_octet(uint32_t bits, bool inside) {
    constexpr uint32_t kOne = dtype_of<XT>::value == SNNF_F16 ? 0x3C00u : 0x3F80u;
    bits = inside ? bits : 0u;
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = ((((bits >> (2 * j)) & 3u) * 0x8001u) & 0x10001u) * kOne;      // bit 0 -> low half, bit 1 -> high half
    return out;
}

template <typename XT>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    using F = typename Frag<XT>::type;
    if constexpr (sizeof(XT) == 2 && dtype_of<XT>::value == SNNF_F16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(F, a), __builtin_bit_cast(F, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(F, a), __builtin_bit_cast(F, b), c, 0, 0, 0);
    }
}

// Waves per workgroup: they split K, so more waves mean more loads in flight per CU.
template <int TT> struct LinWaves { static constexpr int value = TT <= 8 ? 8 : 4; };

// OCF: fragments of 16 output features per workgroup. Two fragments share every activation fragment (half the activation
// traffic per output) at the price of half as many workgroups.
template <typename XT, typename VT, int TT, bool FAST, int OCF>
__global__ __launch_bounds__(LinWaves<TT>::value * 64) void linear_lif_kernel(StepPtrs xs, LinGeom g, const XT* __restrict__ W,
                                                                              const XT* __restrict__ bias,
                                                                              const VT* __restrict__ v_init, XT* __restrict__ spikes,
                                                                              VT* __restrict__ v_out, LifParams lif) {
    constexpr int NW = LinWaves<TT>::value;
    constexpr int TILE_OC = OCF * kTileOC;
    constexpr int OUTS = TILE_OC * kTileM;                    // outputs per workgroup and timestep
    constexpr int PITCH = TILE_OC + 4;                        // floats per row of a partial tile: the 16-byte writes of
                                                              // 8 consecutive lanes (8 rows) then fall into distinct banks
    constexpr int SLAB = kTileM * PITCH;                      // floats per (wave, timestep)
    extern __shared__ __align__(16) float partial[];          // [NW][TT][kTileM][PITCH]
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int oc0 = blockIdx.x * TILE_OC;
    const int m0 = blockIdx.y * kTileM;

    // Operand rows of this lane (clamped: out-of-range rows compute garbage that is never stored).
    const int b_row = min(m0 + (lane & 15), g.M - 1);
    const int koff = (lane >> 4) * 8;
    const XT* wrow[OCF];
#pragma unroll
    for (int f = 0; f < OCF; ++f) wrow[f] = W + static_cast<int64_t>(min(oc0 + f * kTileOC + (lane & 15), g.Fout - 1)) * g.Fin;
    const XT* xrow[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) xrow[t] = static_cast<const XT*>(xs.p[t]) + static_cast<int64_t>(b_row) * g.x_row_stride;

    f32x4 acc[OCF][TT];
#pragma unroll
    for (int f = 0; f < OCF; ++f)
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[f][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // K steps (32 elements of K each) are dealt to the waves in pairs: the two steps of a pair read the two halves of the
    // same 128-byte lines of every operand row back to back. The loads of both steps are issued before the first
    // matrix instruction; the other wave of the SIMD covers the wait.
    u32x4 a0[OCF], a1[OCF], b0[TT], b1[TT];
    auto fetch = [&](int s, u32x4 (&a)[OCF], u32x4 (&b)[TT]) __attribute__((always_inline)) {
        int part = 0;        // fp32 tensors: step s of K part `part` (see LinGeom)
        if constexpr (sizeof(XT) == 4) {
            part = s >= 2 * g.ksteps ? 2 : (s >= g.ksteps ? 1 : 0);
            s -= part * g.ksteps;
        }
        const int k = s * 32 + koff;
#pragma unroll
        for (int f = 0; f < OCF; ++f) a[f] = load_octet<XT, FAST>(wrow[f], k, g.Fin, part == 1);
#pragma unroll
        for (int t = 0; t < TT; ++t) b[t] = load_octet<XT, FAST>(xrow[t], k, g.Fin, part == 2);
    };
    auto multiply = [&](const u32x4 (&a)[OCF], const u32x4 (&b)[TT]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int f = 0; f < OCF; ++f) acc[f][t] = mfma16<XT>(a[f], b[t], acc[f][t]);
    };
    const int all_steps = g.kparts * g.ksteps;
    for (int s = 2 * wave; s < all_steps; s += 2 * NW) {
        const bool second = s + 1 < all_steps;
        fetch(s, a0, b0);
        if (second) fetch(s + 1, a1, b1);
        multiply(a0, b0);
        if (second) multiply(a1, b1);
    }

    // D[i = oc][j = m]: lane holds column j = lane % 16, rows i = 4 * (lane / 16) + r.
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int f = 0; f < OCF; ++f)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                partial[(wave * TT + t) * SLAB + (lane & 15) * PITCH + f * kTileOC + (lane >> 4) * 4 + r] = acc[f][t][r];
    __syncthreads();

    // Output e of the tile = (row e / TILE_OC, feature e % TILE_OC): consecutive threads write consecutive features. The
    // partial sums are added in a fixed order.
    for (int e = threadIdx.x; e < OUTS; e += NW * 64) {
        const int slot = (e / TILE_OC) * PITCH + e % TILE_OC;
        const int m = m0 + e / TILE_OC;
        const int oc = oc0 + e % TILE_OC;
        if (m >= g.M || oc >= g.Fout) continue;
        const float bv = bias != nullptr ? to_float(bias[oc]) : 0.0f;
        const int64_t o = static_cast<int64_t>(m) * g.Fout + oc;
        float v = v_init != nullptr ? to_float(v_init[o]) : 0.0f;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            if (t < g.T) {      // a guard, not a break: a second loop exit keeps the compiler from unrolling over t
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; w += 2) sum += partial[(w * TT + t) * SLAB + slot] + partial[((w + 1) * TT + t) * SLAB + slot];
                const float cur = sum + bv;
                spikes[t * g.spike_step_stride + o] = spike_value<XT>(lif_step(cur, v, lif));
            }
        }
        v_out[o] = from_float<VT>(v);
    }
}

template <typename XT, typename VT, int TT, bool FAST, int OCF>
int launch_one(const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
               void* v_out, const LifParams& lif, hipStream_t stream) {
    constexpr int NW = LinWaves<TT>::value;
    constexpr size_t lds = static_cast<size_t>(NW) * TT * kTileM * (OCF * kTileOC + 4) * sizeof(float);
    static_assert(lds <= 160 * 1024, "partial sums exceed LDS");
    const dim3 grid((g.Fout + OCF * kTileOC - 1) / (OCF * kTileOC), (g.M + kTileM - 1) / kTileM);
    if (grid.y > 65535) return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: M=%d too large", g.M);
    auto kernel = linear_lif_kernel<XT, VT, TT, FAST, OCF>;
    if (lds > 64 * 1024) {
        static const hipError_t raised =
            hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (raised != hipSuccess) return fail(SNNF_ERR_LAUNCH, "snnf_linear_lif: cannot reserve %zu bytes of LDS", lds);
    }
    kernel<<<grid, NW * 64, lds, stream>>>(xs, g, static_cast<const XT*>(W), static_cast<const XT*>(bias),
                                           static_cast<const VT*>(v_init), static_cast<XT*>(spikes), static_cast<VT*>(v_out), lif);
    return check_launch("snnf_linear_lif");
}

// ---------------------------------------------------------------------------------------------------------------
// Staged variant (4 timesteps or more, 16-byte aligned rows, Fin % 8 == 0). Operand fragments fetched straight from
// global memory put the 16 rows of a fragment in 16 adjacent lanes, i.e. 16 different cache lines per 256 bytes
// fetched, and the texture path then delivers about 16 bytes per clock and CU. Here a K slab of 128 elements of every
// operand row (the TM x TT activation rows and the 16 x OCF weight rows of the tile) is fetched with adjacent lanes on
// adjacent 16 bytes, parked in LDS (row pitch 272 bytes: the 16-byte reads of 8 consecutive rows fall into distinct
// banks), and the waves read their fragments from there. Wave w owns activation fragments (w % TG) * TPW ... (a fragment
// is one timestep of 16 rows or two timesteps of 8) and, when fewer than 8 fragment groups leave waves to spare, every
// KSPLIT-th K step of the slab. The next slab's loads are in flight while the
// current one multiplies. The accumulators meet in LDS (aliasing the slab) for the LIF recurrence.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kStagedWaves = 8;
constexpr int kSlabK = 128;                       // K elements per slab = 4 matrix K steps (wider slabs measured no faster once
                                                  // several slabs are in flight; they cost LDS and registers)

// TM rows of the batch per workgroup: 16, or 8 where 16-row tiles would leave half of the compute units idle (a fragment
// of 16 activation rows then holds two timesteps of the 8 rows; the tile stages half the activations per weight row).
template <int TT, int OCF, int SLABK, int TM> struct StagedShape {
    static_assert(TM == 8 || TM == 16, "8 or 16 batch rows per tile");
    static constexpr int FRAGS = TT * TM / 16;                   // activation fragments (16 rows: TM rows of 16 / TM timesteps) per K step
    static constexpr int TPW = FRAGS >= 8 ? 4 : 2;               // fragments per wave: its weight fragments serve all of them (LDS reads per
                                                                 // matrix instruction fall with the size of a wave's register tile)
    static constexpr int TG = FRAGS / TPW;                       // wave groups along time
    static constexpr int KSPLIT = kStagedWaves / TG;             // waves sharing the K steps of a slab
    static_assert(SLABK / 32 >= KSPLIT, "a slab has a K step for every wave of a group");
    static constexpr int ROWS = TT * TM + OCF * kTileOC;         // operand rows per slab
    static constexpr int PITCH_B = SLABK * 2 + 16;               // bytes per operand row in LDS (the 16-byte reads of 8 consecutive rows fall into distinct banks)
    static constexpr int ITEMS = (ROWS * (SLABK / 8) + kStagedWaves * 64 - 1) / (kStagedWaves * 64);   // octets per thread
    static constexpr int RING = ITEMS <= 3 ? 4 : 2;              // slabs in flight per thread (even; ITEMS x 4 registers each, 8 for fp32 storage)
    static constexpr int PITCH = OCF * kTileOC + 4;              // floats per row of an accumulator tile in LDS
    static constexpr size_t slab_bytes = static_cast<size_t>(ROWS) * PITCH_B;
    static constexpr size_t acc_bytes = static_cast<size_t>(KSPLIT) * TT * TM * PITCH * sizeof(float);
    static constexpr size_t lds_bytes = slab_bytes > acc_bytes ? slab_bytes : acc_bytes;
};

// XBITS: the activation rows are rows of bits (byte b of a row = features 8 b ... 8 b + 7, bit j = feature 8 b + j; the row
// stride is in bytes), expanded to 0 / 1 operands where a slab is parked. SBITS: the spikes leave as bits in the same form
// ([T][M][Fout / 8] bytes, the step stride in bytes) instead of elements. Both are the internal layouts of a network executor
// (a convolution on a plane of a few pixels is this matrix product, see snnf_linear_lif_bits).
template <typename XT, typename VT, int TT, int OCF, bool DB, int SLABK, int TM, bool XBITS = false, bool SBITS = false>
__global__ __launch_bounds__(kStagedWaves * 64) void linear_lif_staged_kernel(StepPtrs xs, LinGeom g, const XT* __restrict__ W,
                                                                              const XT* __restrict__ bias,
                                                                              const VT* __restrict__ v_init, XT* __restrict__ spikes,
                                                                              VT* __restrict__ v_out, LifParams lif,
                                                                              float* __restrict__ ws_partial, int* __restrict__ ws_count,
                                                                              int slabs_per_part) {
    using SH = StagedShape<TT, OCF, SLABK, TM>;
    constexpr int kSlabOctets = SLABK / 8;            // 16-byte staging items per operand row
    constexpr int kSlabPitch = SH::PITCH_B;
    constexpr int NT = kStagedWaves * 64;
    constexpr int TILE_OC = OCF * kTileOC;
    constexpr int OUTS = TILE_OC * TM;
    extern __shared__ __align__(16) unsigned char staged_lds[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int oc0 = blockIdx.x * TILE_OC;
    const int m0 = blockIdx.y * TM;

    // The output of this thread in the recurrence at the end (a tile has at most as many as the workgroup has threads):
    // its bias and its membrane are fetched here, so that the recurrence does not begin with a trip to memory.
    static_assert(OUTS <= NT, "one output per thread");
    const int out_m = m0 + tid / TILE_OC, out_oc = oc0 + tid % TILE_OC;
    const bool out_live = tid < OUTS && out_m < g.M && out_oc < g.Fout;
    const int64_t out_index = static_cast<int64_t>(out_live ? out_m : 0) * g.Fout + (out_live ? out_oc : 0);
    const float bv = bias != nullptr ? to_float(bias[out_live ? out_oc : 0]) : 0.0f;
    const float v_first = v_init != nullptr ? to_float(v_init[out_index]) : 0.0f;

    // Staging items of this thread: item i = tid + j * NT is octet i % 16 of operand row i / 16 (NT is a multiple of 16, so
    // the octet is the same for all of a thread's items). Rows beyond M / Fout re-read the last real row; what they produce
    // is never stored.
    const int octet = tid % kSlabOctets;
    constexpr int kRowsPerPass = NT / kSlabOctets;      // operand rows one pass of the workgroup's threads covers
    static_assert(!XBITS || ((TT * TM) % kRowsPerPass == 0 && sizeof(XT) == 2), "a pass holds activation rows or weight rows, not both");
    const XT* item_row[SH::ITEMS];
    uint32_t item_dst[SH::ITEMS];
    bool item_live[SH::ITEMS];
    bool item_is_w[SH::ITEMS];
#pragma unroll
    for (int j = 0; j < SH::ITEMS; ++j) {
        const int row = tid / kSlabOctets + j * (NT / kSlabOctets);
        item_live[j] = row < SH::ROWS;
        const int r = item_live[j] ? row : 0;
        const XT* ptr;
        if (r < TT * TM) {
            const int t = r / TM;
            const void* base = xs.p[0];
#pragma unroll
            for (int u = 1; u < TT; ++u) base = t == u ? xs.p[u] : base;
            if constexpr (XBITS)       // a byte pointer kept in the array of element pointers
                ptr = reinterpret_cast<const XT*>(static_cast<const unsigned char*>(base) + static_cast<int64_t>(min(m0 + r % TM, g.M - 1)) * g.x_row_stride);
            else
                ptr = static_cast<const XT*>(base) + static_cast<int64_t>(min(m0 + r % TM, g.M - 1)) * g.x_row_stride;
        } else {
            ptr = W + static_cast<int64_t>(min(oc0 + r - TT * TM, g.Fout - 1)) * g.Fin;
        }
        item_row[j] = ptr;
        item_is_w[j] = r >= TT * TM;
        item_dst[j] = static_cast<uint32_t>(r * kSlabPitch + octet * 16);
    }

    const int tg = wave % SH::TG;
    const int kp = wave / SH::TG;
    f32x4 acc[OCF][SH::TPW];
#pragma unroll
    for (int f = 0; f < OCF; ++f)
#pragma unroll
        for (int u = 0; u < SH::TPW; ++u) acc[f][u] = f32x4{0.f, 0.f, 0.f, 0.f};

    // RING slabs ahead in registers: a slab's loads have the time of RING - 1 other slabs to arrive, so the loop runs at
    // the rate of its LDS traffic and barriers instead of one memory latency per slab. Every load is unconditional and
    // the ring is walked by a fully unrolled inner loop (static register indices; the compiler can then wait for exactly
    // the oldest slab): the slab count is rounded up to a multiple of RING, and slabs beyond K read zeros (load_octet)
    // and add nothing. DB: two slab buffers in LDS, so that a slab costs one barrier instead of two (writing buffer b for
    // slab s + 1 cannot overtake the reads of slab s - 1, which every wave finished before the barrier of slab s).
    constexpr int RING = SH::RING;
    RawOctet<XT> pre[RING][SH::ITEMS];
    bool pre_inside[RING];
    int pre_part[RING];       // fp32 tensors: the K part a slab belongs to (see LinGeom)
    // K split over workgroups: workgroup z of a tile takes slabs [z * slabs_per_part, ...) (all of them without a split). The
    // slabs of an fp32 tensor's three K parts follow each other: slab s is slab s % unit of part s / unit.
    const int slab0 = static_cast<int>(blockIdx.z) * slabs_per_part;
    const int unit = (g.Fin + SLABK - 1) / SLABK;                        // slabs of one pass over K
    const int slab_end = min(g.kparts * unit, slab0 + slabs_per_part);   // this workgroup's slabs end here: beyond it, zeros
    const int rounds = (slabs_per_part + RING - 1) / RING;
    auto fetch = [&](int slab, int r) __attribute__((always_inline)) {
        int part = 0, real = slab;
        if constexpr (sizeof(XT) == 4) {
            part = slab >= 2 * unit ? 2 : (slab >= unit ? 1 : 0);
            real = slab - part * unit;
        }
        pre_part[r] = part;
        const int k = real * SLABK + octet * 8;
        pre_inside[r] = slab < slab_end && k < g.Fin;
        const int ks = pre_inside[r] ? k : 0;
#pragma unroll
        for (int j = 0; j < SH::ITEMS; ++j) {
            if (XBITS && j * kRowsPerPass < TT * TM)       // one byte = the octet's eight features
                pre[r][j].lo[0] = reinterpret_cast<const unsigned char*>(item_row[j])[ks >> 3];
            else
                pre[r][j] = load_raw_octet<XT>(item_row[j] + ks);   // items beyond the rows re-read row 0
        }
    };
    // Fragment addresses in the slab: lane = 16 q + r reads K elements 8 q .. 8 q + 7 of row r of its fragment.
    const uint32_t frag_off = static_cast<uint32_t>((lane & 15) * kSlabPitch + (lane >> 4) * 16);
#pragma unroll
    for (int r = 0; r < RING; ++r) {
        fetch(slab0 + r, r);
        __builtin_amdgcn_sched_barrier(0);      // oldest slab first, as in the loop: its wait then leaves the others in flight
    }
    // A slab parked in LDS from the ring, and this wave's K steps of a parked slab (every KSPLIT-th), four at a time: their
    // operand reads go out together.
    auto park = [&](int r, unsigned char* buf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < SH::ITEMS; ++j)
            if (item_live[j]) {
                if (XBITS && j * kRowsPerPass < TT * TM)
                    *reinterpret_cast<u32x4*>(buf + item_dst[j]) = expand_bit_octet<XT>(pre[r][j].lo[0], pre_inside[r]);
                else
                    *reinterpret_cast<u32x4*>(buf + item_dst[j]) = finish_octet<XT>(pre[r][j], pre_inside[r], pre_part[r] == (item_is_w[j] ? 1 : 2));
            }
    };
    auto multiply = [&](const unsigned char* buf) __attribute__((always_inline)) {
        constexpr int OWN = SLABK / 32 / SH::KSPLIT;
        const unsigned char* own = buf + frag_off + (kp % SH::KSPLIT) * 64;
#pragma unroll
        for (int i0 = 0; i0 < OWN; i0 += 4) {
            u32x4 a[4][OCF], b[4][SH::TPW];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i0 + i < OWN) {
                    const int off = (i0 + i) * SH::KSPLIT * 64;
#pragma unroll
                    for (int f = 0; f < OCF; ++f) a[i][f] = *reinterpret_cast<const u32x4*>(own + (TT * TM + f * kTileOC) * kSlabPitch + off);
#pragma unroll
                    for (int u = 0; u < SH::TPW; ++u) b[i][u] = *reinterpret_cast<const u32x4*>(own + (tg * SH::TPW + u) * 16 * kSlabPitch + off);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i0 + i < OWN) {
#pragma unroll
                    for (int u = 0; u < SH::TPW; ++u)
#pragma unroll
                        for (int f = 0; f < OCF; ++f) acc[f][u] = mfma16<XT>(a[i][f], b[i][u], acc[f][u]);
                }
            }
        }
    };
    // Parking slab s + 1 (in the other buffer) ahead of the multiplication of slab s, so that a slab's barrier does not wait
    // for its writes, measured slower (64 rows x 8 timesteps 2048 -> 1024: 10.0 -> 10.4 us, 16 rows 25088 -> 4096: 63 -> 76):
    // the wait for the loads of s + 1 then stands before the work on s.
    for (int round = 0; round < rounds; ++round) {
#pragma unroll
        for (int r = 0; r < RING; ++r) {
            const int slab = slab0 + round * RING + r;
            unsigned char* buf = staged_lds + (DB ? (r & 1) * SH::slab_bytes : 0);      // RING is even
            park(r, buf);
            __syncthreads();
            fetch(slab + RING, r);
            multiply(buf);
            if (!DB) __syncthreads();
        }
    }
    if (DB) __syncthreads();

    // Accumulators -> LDS as [K part][t][m][PITCH] (row t * TM + m is row (t * TM + m) % 16 of fragment (t * TM + m) / 16);
    // D[i = oc][j = row]: lane holds column j = lane % 16, rows 4 (lane / 16) + r.
    float* partial = reinterpret_cast<float*>(staged_lds);
    constexpr int SLAB_F = TM * SH::PITCH;
#pragma unroll
    for (int u = 0; u < SH::TPW; ++u)
#pragma unroll
        for (int f = 0; f < OCF; ++f)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                partial[((kp * SH::FRAGS + tg * SH::TPW + u) * 16 + (lane & 15)) * SH::PITCH + f * kTileOC + (lane >> 4) * 4 + r] = acc[f][u][r];
    __syncthreads();

    // K split over workgroups: every workgroup of a tile leaves its sums in the workspace and counts itself in; the one
    // that arrives last adds all parts in the order of their K ranges (so the result does not depend on who was last)
    // and runs the recurrence. It leaves the counter at zero for the next launch. The sums and the counter travel as
    // device-scope atomic stores, loads and adds (relaxed): those go through to memory, past the L2 caches of the chip's
    // partitions, which do not see each other's lines. A device-scope fence would do too, but it writes back a whole L2
    // per wave that executes it and costs more than the kernel. Order: every thread waits until its own write-through
    // stores have been acknowledged (an explicit wait on the vector-memory counter: neither a workgroup barrier nor a
    // workgroup-scope fence implies one for global stores), then the workgroup barrier, then one thread counts the
    // workgroup in. The last arriver's loads are device-scope atomic loads issued after it has read the counter.
    const int parts = static_cast<int>(gridDim.z);
    const int tile = static_cast<int>(blockIdx.y * gridDim.x + blockIdx.x);
    if (parts > 1) {
        __shared__ int arrived_last;
        float* __restrict__ mine = ws_partial + (static_cast<int64_t>(tile) * parts + blockIdx.z) * (TT * OUTS);
        for (int e = tid; e < OUTS; e += NT) {
            const int slot = (e / TILE_OC) * SH::PITCH + e % TILE_OC;
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < SH::KSPLIT; ++w) sum += partial[(w * TT + t) * SLAB_F + slot];
                __hip_atomic_store(mine + t * OUTS + e, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this thread's partial sums have reached memory
        __syncthreads();
        if (tid == 0) {
            const int before = __hip_atomic_fetch_add(ws_count + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            arrived_last = before == parts - 1 ? 1 : 0;
            if (arrived_last) __hip_atomic_store(ws_count + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!arrived_last) return;
    }

    if (SBITS ? tid < OUTS : out_live) {      // SBITS: whole waves, for the ballot (OUTS is a multiple of 64)
        const int e = tid;
        const int slot = (e / TILE_OC) * SH::PITCH + e % TILE_OC;
        float v = v_first;
        const float* __restrict__ all = ws_partial + static_cast<int64_t>(tile) * parts * (TT * OUTS) + e;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            if (t < g.T) {      // a guard, not a break: a second loop exit keeps the compiler from unrolling over t
                float sum = 0.0f;
                if (parts > 1) {
                    for (int z = 0; z < parts; ++z) sum += __hip_atomic_load(all + (static_cast<int64_t>(z) * TT + t) * OUTS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
#pragma unroll
                    for (int w = 0; w < SH::KSPLIT; ++w) sum += partial[(w * TT + t) * SLAB_F + slot];
                }
                const float cur = sum + bv;
                const bool fired = lif_step(cur, v, lif);
                if constexpr (SBITS) {
                    // Lane l of the wave holds feature oc0 + l % TILE_OC (a multiple of 8 apart from l % 8): byte l / 8 of the ballot.
                    const uint64_t fired_lanes = __ballot(fired && out_live);
                    if ((lane & 7) == 0 && out_live)
                        reinterpret_cast<unsigned char*>(spikes)[t * g.spike_step_stride + static_cast<int64_t>(out_m) * (g.Fout >> 3) + (out_oc >> 3)] =
                            static_cast<unsigned char>(fired_lanes >> lane);
                } else {
                    spikes[t * g.spike_step_stride + out_index] = spike_value<XT>(fired);
                }
            }
        }
        if (v_out != nullptr && out_live) v_out[out_index] = from_float<VT>(v);
    }
}

// Workspace of the split: one counter per tile (zero between launches), then [tile][part][t][16 x TILE_OC] sums.
struct LinWorkspace {
    void* base;
    size_t bytes;
};
constexpr size_t kLinCounterBytes = 64 * 1024;     // 16384 tiles
constexpr int kLinLongK = 96;                      // K slabs from which two K parts of 16-row tiles beat 8-row tiles (see linear_half_row_tiles)

template <typename XT, typename VT, int TT, int OCF, bool DB, int SLABK, int TM, bool XBITS = false, bool SBITS = false>
int launch_staged_db(dim3 grid, int slabs_per_part, const LinWorkspace& ws, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias,
                     const void* v_init, void* spikes, void* v_out, const LifParams& lif, hipStream_t stream) {
    using SH = StagedShape<TT, OCF, SLABK, TM>;
    constexpr size_t lds = DB ? 2 * SH::slab_bytes : SH::lds_bytes;
    static_assert(lds <= 160 * 1024 && SH::acc_bytes <= lds, "slabs exceed LDS");
    auto kernel = linear_lif_staged_kernel<XT, VT, TT, OCF, DB, SLABK, TM, XBITS, SBITS>;
    if (lds > 64 * 1024) {
        static const hipError_t raised = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (raised != hipSuccess) return fail(SNNF_ERR_LAUNCH, "snnf_linear_lif: cannot reserve %zu bytes of LDS", lds);
    }
    kernel<<<grid, kStagedWaves * 64, lds, stream>>>(xs, g, static_cast<const XT*>(W), static_cast<const XT*>(bias),
                                                     static_cast<const VT*>(v_init), static_cast<XT*>(spikes),
                                                     static_cast<VT*>(v_out), lif,
                                                     reinterpret_cast<float*>(static_cast<char*>(ws.base) + kLinCounterBytes),
                                                     static_cast<int*>(ws.base), slabs_per_part);
    return check_launch("snnf_linear_lif");
}

// Parts the K dimension of a tile is split into: two, for a layer with a long K whose tiles leave half of the compute
// units idle (the classifier layers at small batch), when the workspace takes it. Splitting costs three trips to memory
// at the end of a tile; measured, it pays from K = 4096 on (4096 -> 4096 at 16 rows: 16.5 -> 13.9 us, 25088 -> 4096:
// 75 -> 47 us) and more than two parts gain nothing.
inline int linear_split_parts(int64_t tiles, int unit_slabs, size_t part_bytes, size_t ws_bytes) {
    if (tiles > static_cast<int64_t>(kLinCounterBytes / sizeof(int)) || tiles * 2 > compute_units() || unit_slabs < 32) return 1;
    if (ws_bytes < kLinCounterBytes + 2 * part_bytes * static_cast<size_t>(tiles)) return 1;
    return 2;
}

template <typename XT, typename VT, int TT, int OCF, int TM = kTileM, int SLABK = kSlabK, bool XBITS = false, bool SBITS = false>
int launch_staged(const LinWorkspace& ws, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
                  void* v_out, const LifParams& lif, hipStream_t stream) {
    dim3 grid((g.Fout + OCF * kTileOC - 1) / (OCF * kTileOC), (g.M + TM - 1) / TM);
    if (grid.y > 65535) return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: M=%d too large", g.M);
    const int unit_slabs = g.kparts * ((g.Fin + SLABK - 1) / SLABK);          // all K parts of an fp32 tensor
    const int64_t tiles = static_cast<int64_t>(grid.x) * grid.y;
    const size_t part_bytes = static_cast<size_t>(TT) * OCF * kTileOC * TM * sizeof(float);
    int parts = ws.base != nullptr ? linear_split_parts(tiles, unit_slabs * (SLABK / kSlabK), part_bytes, ws.bytes) : 1;
    const int unit_slabs_per_part = (unit_slabs + parts - 1) / parts;
    using SH = StagedShape<TT, OCF, SLABK, TM>;
    parts = (unit_slabs + unit_slabs_per_part - 1) / unit_slabs_per_part;      // no empty part
    grid.z = parts;
    // Two slab buffers where a CU gets one workgroup anyway (they would cost occupancy otherwise) and both fit LDS.
    constexpr bool can_double = 2 * SH::slab_bytes <= 160 * 1024;
    if constexpr (can_double) {
        if (tiles * parts <= compute_units())
            return launch_staged_db<XT, VT, TT, OCF, true, SLABK, TM, XBITS, SBITS>(grid, unit_slabs_per_part, ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    }
    return launch_staged_db<XT, VT, TT, OCF, false, SLABK, TM, XBITS, SBITS>(grid, unit_slabs_per_part, ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

// Tiles of 8 batch rows instead of 16 (a workgroup then stages 8 x T activation rows per slab for its 32 weight rows):
// for batches of up to 8 rows, whose tiles of 16 would stage every row twice, and where tiles of 16 rows give workgroups
// to at most half of the compute units. Measured at 8 timesteps, 16-bit tensors (16 -> 8 rows): 64 rows 2048 -> 1024
// 13.5 -> 10.5 us (16 timesteps: 24.8 -> 16.8), 24 rows 1024 -> 2048 9.1 -> 7.4, 16 rows 4096 -> 4096 20.0 -> 16.8 (against
// 16-row tiles with K split in two), 1 row 25088 -> 4096 61.9 -> 43.5; slower where 16-row tiles fill the chip (128 rows
// 2048 -> 1024 15.3 -> 18.7) and for the longest K, where two K parts of 16-row tiles read every weight once and two
// 8-row tiles read it twice (16 rows 25088 -> 4096: 65 -> 71 with a workspace).
inline bool linear_half_row_tiles(const LinWorkspace& ws, const LinGeom& g) {
    if (g.M <= 8) return true;
    const int64_t oc_tiles = g.Fout % (2 * kTileOC) == 0 ? g.Fout / (2 * kTileOC) : (g.Fout + kTileOC - 1) / kTileOC;
    if (oc_tiles * ((g.M + kTileM - 1) / kTileM) * 2 > compute_units()) return false;
    const int unit_slabs = g.kparts * ((g.Fin + kSlabK - 1) / kSlabK);
    if (ws.base == nullptr || unit_slabs < 32) return true;                  // K is not split either way
    if (oc_tiles * ((g.M + 7) / 8) * 2 <= compute_units()) return true;      // tiles of 8 rows split K as well
    // 16-row tiles in two K parts or 8-row tiles unsplit: up to 4 timesteps the split wins (16 rows 4096 -> 4096: 13.6
    // against 14.0 us), beyond that only for the longest K.
    return g.T > 4 && unit_slabs < kLinLongK;
}

template <typename XT, typename VT, int OCF, int TM>
int launch_staged_tt(const LinWorkspace& ws, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
                     void* v_out, const LifParams& lif, hipStream_t stream) {
    // 4 timesteps of 8 rows are two fragments: their eight waves split a slab of 8 K steps. Narrow tiles of 8 rows take
    // slabs of 8 K steps too: with one weight fragment a wave has too little to do per barrier otherwise (8 timesteps,
    // 16 rows, 2048 -> 1024: 8.9 -> 7.9 us; 8 rows 25088 -> 1000: 39.5 -> 33.6); wide tiles are slower that way (64 rows
    // 2048 -> 1024: 10.1 -> 11.0 us).
    constexpr int kWide = (TM == 8 && OCF == 1) ? 2 * kSlabK : kSlabK;
    if (g.T <= 4) return launch_staged<XT, VT, 4, OCF, TM, TM == 8 ? 2 * kSlabK : kSlabK>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 8) return launch_staged<XT, VT, 8, OCF, TM, kWide>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    return launch_staged<XT, VT, 16, OCF, TM, kWide>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

template <typename XT, typename VT, bool FAST>
int launch_tt(const LinWorkspace& ws, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
              void* v_out, const LifParams& lif, hipStream_t stream) {
    if constexpr (FAST) {
        if (g.T > 2) {
            // Two feature fragments per workgroup (half the activation traffic) when that still leaves at least 128 workgroups.
            const bool half_rows = linear_half_row_tiles(ws, g);
            const int tm = half_rows ? 8 : kTileM;
            const bool wide = g.Fout % (2 * kTileOC) == 0 && static_cast<int64_t>(g.Fout / (2 * kTileOC)) * ((g.M + tm - 1) / tm) >= 128;
            if (half_rows) {
                if (wide) return launch_staged_tt<XT, VT, 2, 8>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
                return launch_staged_tt<XT, VT, 1, 8>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
            }
            if (wide) return launch_staged_tt<XT, VT, 2, kTileM>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
            return launch_staged_tt<XT, VT, 1, kTileM>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
        }
    }
    if (g.T <= 1) return launch_one<XT, VT, 1, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 2) return launch_one<XT, VT, 2, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 4) return launch_one<XT, VT, 4, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 8) return launch_one<XT, VT, 8, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    return launch_one<XT, VT, 16, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

// The internal-layout forms: spikes out as bits, activation rows as elements or as bits; wide tiles (Fout % 32 == 0), 3 to 8
// timesteps, fp32 membrane.
template <typename XT, bool XBITS>
int launch_bits(const LinWorkspace& ws, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
                void* v_out, const LifParams& lif, hipStream_t stream) {
    if (linear_half_row_tiles(ws, g)) {
        if (g.T <= 4) return launch_staged<XT, float, 4, 2, 8, 2 * kSlabK, XBITS, true>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
        return launch_staged<XT, float, 8, 2, 8, kSlabK, XBITS, true>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    }
    if (g.T <= 4) return launch_staged<XT, float, 4, 2, kTileM, kSlabK, XBITS, true>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    return launch_staged<XT, float, 8, 2, kTileM, kSlabK, XBITS, true>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

template <typename XT, typename VT>
int launch(bool fast, const LinWorkspace& ws, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init,
           void* spikes, void* v_out, const LifParams& lif, hipStream_t stream) {
    return fast ? launch_tt<XT, VT, true>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream)
                : launch_tt<XT, VT, false>(ws, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

}  // namespace
}  // namespace snnf

extern "C" size_t snnf_linear_lif_workspace_bytes(int T, int M, int Fin, int Fout) {
    using namespace snnf;
    if (T < 3 || M < 1 || Fin < 1 || Fout < 1) return 0;      // one or two timesteps run on the kernel without staging
    int tt = 4;
    while (tt < T && tt < SNNF_MAX_T_PER_LAUNCH) tt *= 2;
    const int64_t m_tiles = (M + kTileM - 1) / kTileM;
    const int64_t tiles = ((Fout + kTileOC - 1) / kTileOC) * m_tiles;          // the narrow tiling has the most tiles
    const int all_slabs = (Fin + kSlabK - 1) / kSlabK;
    if (tiles > compute_units() || all_slabs < 32 || tiles > static_cast<int64_t>(kLinCounterBytes / sizeof(int))) return 0;
    const int64_t parts = 2;
    // Sums of one part of one tile: TT x 16 rows x 16 features x 4 bytes for the narrow tiling, twice that for half as many wide tiles.
    const size_t sums = static_cast<size_t>(tiles) * parts * tt * kTileM * kTileOC * sizeof(float);
    return kLinCounterBytes + sums;
}

static int linear_lif_impl(const char* who, const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                           const void* weight, const void* bias, int Fout, int w_dtype, const void* v_init,
                           int v_dtype, void* spikes, int64_t spike_step_stride, void* v_out, float v_threshold,
                           float v_reset, float tau, void* workspace, size_t workspace_bytes, void* stream);

extern "C" int snnf_linear_lif(const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                               const void* weight, const void* bias, int Fout, int w_dtype, const void* v_init,
                               int v_dtype, void* spikes, int64_t spike_step_stride, void* v_out, float v_threshold,
                               float v_reset, float tau, void* stream) {
    return linear_lif_impl("snnf_linear_lif", xs, T, M, Fin, x_row_stride, x_dtype, weight, bias, Fout, w_dtype, v_init, v_dtype, spikes,
                           spike_step_stride, v_out, v_threshold, v_reset, tau, nullptr, 0, stream);
}

extern "C" int snnf_linear_lif_ws(const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                                  const void* weight, const void* bias, int Fout, int w_dtype, const void* v_init,
                                  int v_dtype, void* spikes, int64_t spike_step_stride, void* v_out, float v_threshold,
                                  float v_reset, float tau, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace snnf;
    if (workspace != nullptr && !aligned_to(workspace, 256))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_ws: workspace must be 256-byte aligned");
    return linear_lif_impl("snnf_linear_lif_ws", xs, T, M, Fin, x_row_stride, x_dtype, weight, bias, Fout, w_dtype, v_init, v_dtype, spikes,
                           spike_step_stride, v_out, v_threshold, v_reset, tau, workspace, workspace != nullptr ? workspace_bytes : 0, stream);
}

static int linear_lif_impl(const char* who, const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                           const void* weight, const void* bias, int Fout, int w_dtype, const void* v_init,
                           int v_dtype, void* spikes, int64_t spike_step_stride, void* v_out, float v_threshold,
                           float v_reset, float tau, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace snnf;
    (void)who;
    const LinWorkspace ws = {workspace, workspace_bytes};
    if (xs == nullptr || weight == nullptr || spikes == nullptr || v_out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif: xs, weight, spikes and v_out must be non-null");
    if (T < 1 || M < 1 || Fin < 1 || Fout < 1 || x_row_stride < Fin)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif: T=%d M=%d Fin=%d Fout=%d x_row_stride=%lld", T, M, Fin,
                    Fout, (long long)x_row_stride);
    if (!valid_dtype(x_dtype) || !valid_dtype(v_dtype) || !valid_dtype(w_dtype))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif: unknown dtype code");
    if (w_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: unsupported_dtype: weight/bias dtype must match x");
    if (v_dtype != SNNF_F32 && v_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: unsupported_dtype: membrane dtype must be fp32 or the activation dtype");
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: unsupported_tau: tau must be nonzero");
    for (int t = 0; t < T; ++t)
        if (xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif: xs[%d] is null", t);

    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    const int xsize = dtype_size(x_dtype);
    hipStream_t hs = as_stream(stream);
    const int per16 = 16 / xsize;

    for (int t0 = 0; t0 < T; t0 += SNNF_MAX_T_PER_LAUNCH) {
        const int tw = (T - t0) < SNNF_MAX_T_PER_LAUNCH ? (T - t0) : SNNF_MAX_T_PER_LAUNCH;
        int tt = 1;
        while (tt < tw) tt *= 2;
        StepPtrs ptrs = {};
        bool fast = Fin % 8 == 0 && x_row_stride % per16 == 0 && aligned_to(weight, 16);
        for (int t = 0; t < tt; ++t) {
            ptrs.p[t] = xs[t0 + (t < tw ? t : 0)];  // padded steps re-read step 0 and are never stored
            fast = fast && aligned_to(ptrs.p[t], 16);
        }
        LinGeom g;
        g.T = tw;
        g.M = M;
        g.Fin = Fin;
        g.Fout = Fout;
        g.x_row_stride = x_row_stride;
        g.spike_step_stride = spike_step_stride;
        g.ksteps = (Fin + 31) / 32;
        g.kparts = x_dtype == SNNF_F32 ? 3 : 1;
        const void* vi = t0 == 0 ? v_init : v_out;
        void* sp = static_cast<char*>(spikes) + static_cast<int64_t>(t0) * spike_step_stride * xsize;
        int rc;
        if (x_dtype == SNNF_F32) rc = launch<float, float>(fast, ws, ptrs, g, weight, bias, vi, sp, v_out, lif, hs);
        else if (x_dtype == SNNF_BF16)
            rc = v_dtype == SNNF_F32 ? launch<bf16_t, float>(fast, ws, ptrs, g, weight, bias, vi, sp, v_out, lif, hs)
                                     : launch<bf16_t, bf16_t>(fast, ws, ptrs, g, weight, bias, vi, sp, v_out, lif, hs);
        else
            rc = v_dtype == SNNF_F32 ? launch<f16_t, float>(fast, ws, ptrs, g, weight, bias, vi, sp, v_out, lif, hs)
                                     : launch<f16_t, f16_t>(fast, ws, ptrs, g, weight, bias, vi, sp, v_out, lif, hs);
        if (rc != SNNF_OK) return rc;
    }
    return SNNF_OK;
}

extern "C" int snnf_linear_lif_bits(const void* const* xs, int x_bits, int T, int M, int Fin, int64_t x_row_stride, int dtype,
                                    const void* weight, const void* bias, int Fout, const void* v_init, void* spike_bits,
                                    int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset, float tau,
                                    void* workspace, size_t workspace_bytes, void* stream) {
    using namespace snnf;
    if (xs == nullptr || weight == nullptr || spike_bits == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: xs, weight and spike_bits must be non-null");
    if (T < 1 || M < 1 || Fin < 1 || Fout < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: T=%d M=%d Fin=%d Fout=%d", T, M, Fin, Fout);
    if (dtype != SNNF_BF16 && dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif_bits: unsupported_dtype: bfloat16 or float16 weights (and activation elements)");
    if (T < 3 || T > 8)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif_bits: unsupported_window: 3 to 8 timesteps per call, got %d", T);
    if (Fin % 8 != 0 || Fout % 32 != 0)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif_bits: unsupported_shape: Fin %% 8 and Fout %% 32 must be 0, got %d -> %d", Fin, Fout);
    if (x_row_stride < (x_bits ? Fin / 8 : Fin) || (!x_bits && x_row_stride % 8 != 0))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: x_row_stride=%lld (bytes for rows of bits, elements in multiples of 8 otherwise)",
                    (long long)x_row_stride);
    if (spike_step_stride < static_cast<int64_t>(M) * (Fout / 8))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: spike_step_stride=%lld bytes is less than a step's M * Fout / 8", (long long)spike_step_stride);
    if (!aligned_to(weight, 16)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: weight must be 16-byte aligned");
    if (workspace != nullptr && !aligned_to(workspace, 256))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: workspace must be 256-byte aligned");
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif_bits: unsupported_tau: tau must be nonzero");
    const int tt = T <= 4 ? 4 : 8;
    StepPtrs ptrs = {};
    for (int t = 0; t < tt; ++t) {
        ptrs.p[t] = xs[t < T ? t : 0];      // padded steps re-read step 0 and are never stored
        if (ptrs.p[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: xs[%d] is null", t);
        if (!x_bits && !aligned_to(ptrs.p[t], 16)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_linear_lif_bits: xs[%d] must be 16-byte aligned", t);
    }
    LinGeom g;
    g.T = T;
    g.M = M;
    g.Fin = Fin;
    g.Fout = Fout;
    g.x_row_stride = x_row_stride;
    g.spike_step_stride = spike_step_stride;
    g.ksteps = (Fin + 31) / 32;
    g.kparts = 1;
    const LinWorkspace ws = {workspace, workspace != nullptr ? workspace_bytes : 0};
    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    hipStream_t hs = as_stream(stream);
    if (dtype == SNNF_BF16)
        return x_bits ? launch_bits<bf16_t, true>(ws, ptrs, g, weight, bias, v_init, spike_bits, v_out, lif, hs)
                      : launch_bits<bf16_t, false>(ws, ptrs, g, weight, bias, v_init, spike_bits, v_out, lif, hs);
    return x_bits ? launch_bits<f16_t, true>(ws, ptrs, g, weight, bias, v_init, spike_bits, v_out, lif, hs)
                  : launch_bits<f16_t, false>(ws, ptrs, g, weight, bias, v_init, spike_bits, v_out, lif, hs);
}
