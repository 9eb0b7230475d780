// Temporal Linear + LIF on the matrix cores: out^T[Fout, T*M] = W[Fout, Fin] . x^T, LIF recurrence in the epilogue.
//
// Both operands are K-contiguous in memory (x rows and W rows), which is the per-lane operand order of
// v_mfma_f32_16x16x32 (8 consecutive k per lane). All T timesteps of a row tile share one weight fragment (the weight is
// streamed once per workgroup, not once per timestep), and each thread runs the LIF recurrence over T for its (row,
// output feature) pair with the membrane in a register. Two kernels: the staged one (4 timesteps or more, aligned rows)
// moves K slabs of all operand rows through LDS with coalesced loads; the direct one (everything else) loads fragments
// straight from global memory, its 8 (beyond 8 timesteps, 4) waves splitting K in pairs of K steps with partial sums
// meeting in LDS.
#include "snnf_common.h"

namespace snnf {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileOC = 16;   // output features per workgroup
constexpr int kTileM = 16;    // rows per workgroup (per timestep)

struct LinGeom {
    int T, M, Fin, Fout;
    int64_t x_row_stride;      // elements
    int64_t spike_step_stride; // elements
    int ksteps;                // ceil(Fin / 32)
};

// Eight consecutive K elements of one row as a matrix-core operand (bf16 for fp32/bf16 storage, fp16 for fp16 storage).
template <typename XT> struct Frag;
template <> struct Frag<bf16_t> { using type = bf16x8; };
template <> struct Frag<float> { using type = bf16x8; };
template <> struct Frag<f16_t> { using type = f16x8; };

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return float_to_bf16_bits(lo) | (float_to_bf16_bits(hi) << 16);
}

// Loads k .. k+7 of `row`; elements at or beyond `kmax` read as zero. FAST requires 16-byte aligned rows and kmax % 8 == 0
// and is branch-free (an octet beyond kmax re-reads the row's first one and is zeroed): a branch around a load would make
// the compiler wait for every load before it issues the next.
template <typename XT, bool FAST>
__device__ __forceinline__ u32x4 load_octet(const XT* __restrict__ row, int k, int kmax) {
    u32x4 out = {0u, 0u, 0u, 0u};
    if constexpr (FAST) {
        const bool inside = k < kmax;
        const XT* __restrict__ src = row + (inside ? k : 0);
        if constexpr (sizeof(XT) == 2) {
            out = *reinterpret_cast<const u32x4*>(src);
        } else {
            const f32x4 a = *reinterpret_cast<const f32x4*>(src);
            const f32x4 b = *reinterpret_cast<const f32x4*>(src + 4);
            out[0] = pack_bf16x2(a[0], a[1]);
            out[1] = pack_bf16x2(a[2], a[3]);
            out[2] = pack_bf16x2(b[0], b[1]);
            out[3] = pack_bf16x2(b[2], b[3]);
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
            out[j] = pack_bf16x2(lo, hi);
        }
    }
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
        const int k = s * 32 + koff;
#pragma unroll
        for (int f = 0; f < OCF; ++f) a[f] = load_octet<XT, FAST>(wrow[f], k, g.Fin);
#pragma unroll
        for (int t = 0; t < TT; ++t) b[t] = load_octet<XT, FAST>(xrow[t], k, g.Fin);
    };
    auto multiply = [&](const u32x4 (&a)[OCF], const u32x4 (&b)[TT]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int f = 0; f < OCF; ++f) acc[f][t] = mfma16<XT>(a[f], b[t], acc[f][t]);
    };
    for (int s = 2 * wave; s < g.ksteps; s += 2 * NW) {
        const bool second = s + 1 < g.ksteps;
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
            if (t >= g.T) break;
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w += 2) sum += partial[(w * TT + t) * SLAB + slot] + partial[((w + 1) * TT + t) * SLAB + slot];
            const float cur = sum + bv;
            spikes[t * g.spike_step_stride + o] = spike_value<XT>(lif_step(cur, v, lif));
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
// operand row (the 16 x TT activation rows and the 16 x OCF weight rows of the tile) is fetched with adjacent lanes on
// adjacent 16 bytes, parked in LDS (row pitch 272 bytes: the 16-byte reads of 8 consecutive rows fall into distinct
// banks), and the waves read their fragments from there. Wave w owns timesteps (w % TG) * TPW ... and, when fewer than 8
// timesteps leave waves to spare, every KSPLIT-th K step of the slab. The next slab's loads are in flight while the
// current one multiplies. The accumulators meet in LDS (aliasing the slab) for the LIF recurrence.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kStagedWaves = 8;
constexpr int kSlabK = 128;                       // K elements per slab = 4 matrix K steps (256: +6 % on one workgroup per
                                                  // CU, -25 % where several fit a CU)
constexpr int kSlabOctets = kSlabK / 8;           // 16-byte staging items per operand row
constexpr int kSlabPitch = kSlabK * 2 + 16;       // bytes per operand row in LDS

template <int TT, int OCF> struct StagedShape {
    static constexpr int TPW = TT >= 8 ? TT / 8 : 1;            // timesteps per wave
    static constexpr int TG = TT / TPW;                          // wave groups along time
    static constexpr int KSPLIT = kStagedWaves / TG;             // waves sharing the K steps of a slab
    static constexpr int ROWS = TT * kTileM + OCF * kTileOC;     // operand rows per slab
    static constexpr int ITEMS = (ROWS * (kSlabK / 8) + kStagedWaves * 64 - 1) / (kStagedWaves * 64);   // octets per thread
    static constexpr int PITCH = OCF * kTileOC + 4;              // floats per row of an accumulator tile in LDS
    static constexpr size_t slab_bytes = static_cast<size_t>(ROWS) * kSlabPitch;
    static constexpr size_t acc_bytes = static_cast<size_t>(KSPLIT) * TT * kTileM * PITCH * sizeof(float);
    static constexpr size_t lds_bytes = slab_bytes > acc_bytes ? slab_bytes : acc_bytes;
};

template <typename XT, typename VT, int TT, int OCF, bool DB>
__global__ __launch_bounds__(kStagedWaves * 64) void linear_lif_staged_kernel(StepPtrs xs, LinGeom g, const XT* __restrict__ W,
                                                                              const XT* __restrict__ bias,
                                                                              const VT* __restrict__ v_init, XT* __restrict__ spikes,
                                                                              VT* __restrict__ v_out, LifParams lif) {
    using SH = StagedShape<TT, OCF>;
    constexpr int NT = kStagedWaves * 64;
    constexpr int TILE_OC = OCF * kTileOC;
    constexpr int OUTS = TILE_OC * kTileM;
    extern __shared__ __align__(16) unsigned char staged_lds[];
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int oc0 = blockIdx.x * TILE_OC;
    const int m0 = blockIdx.y * kTileM;

    // Staging items of this thread: item i = tid + j * NT is octet i % 16 of operand row i / 16 (NT is a multiple of 16, so
    // the octet is the same for all of a thread's items). Rows beyond M / Fout re-read the last real row; what they produce
    // is never stored.
    const int octet = tid % kSlabOctets;
    const XT* item_row[SH::ITEMS];
    uint32_t item_dst[SH::ITEMS];
    bool item_live[SH::ITEMS];
#pragma unroll
    for (int j = 0; j < SH::ITEMS; ++j) {
        const int row = tid / kSlabOctets + j * (NT / kSlabOctets);
        item_live[j] = row < SH::ROWS;
        const int r = item_live[j] ? row : 0;
        const XT* ptr;
        if (r < TT * kTileM) {
            const int t = r / kTileM;
            const void* base = xs.p[0];
#pragma unroll
            for (int u = 1; u < TT; ++u) base = t == u ? xs.p[u] : base;
            ptr = static_cast<const XT*>(base) + static_cast<int64_t>(min(m0 + r % kTileM, g.M - 1)) * g.x_row_stride;
        } else {
            ptr = W + static_cast<int64_t>(min(oc0 + r - TT * kTileM, g.Fout - 1)) * g.Fin;
        }
        item_row[j] = ptr;
        item_dst[j] = static_cast<uint32_t>(r * kSlabPitch + octet * 16);
    }

    const int tg = wave % SH::TG;
    const int kp = wave / SH::TG;
    f32x4 acc[OCF][SH::TPW];
#pragma unroll
    for (int f = 0; f < OCF; ++f)
#pragma unroll
        for (int u = 0; u < SH::TPW; ++u) acc[f][u] = f32x4{0.f, 0.f, 0.f, 0.f};

    // One slab ahead in registers (deeper rings measured slower: the slab loop is bound by LDS traffic and its barriers,
    // not by the latency of the loads). DB: two slab buffers in LDS, so that a slab costs one barrier instead of two
    // (writing buffer b for slab s + 1 cannot overtake the reads of slab s - 1, which every wave finished before the
    // barrier of slab s).
    u32x4 pre[SH::ITEMS];
    auto fetch = [&](int slab) __attribute__((always_inline)) {
        const int k = slab * kSlabK + octet * 8;
#pragma unroll
        for (int j = 0; j < SH::ITEMS; ++j)
            if (item_live[j]) pre[j] = load_octet<XT, true>(item_row[j], k, g.Fin);
    };
    const int nslabs = (g.Fin + kSlabK - 1) / kSlabK;
    // Fragment addresses in the slab: lane = 16 q + r reads K elements 8 q .. 8 q + 7 of row r of its fragment.
    const uint32_t frag_off = static_cast<uint32_t>((lane & 15) * kSlabPitch + (lane >> 4) * 16);
    fetch(0);
    for (int slab = 0; slab < nslabs; ++slab) {
        unsigned char* buf = staged_lds + (DB ? (slab & 1) * SH::slab_bytes : 0);
#pragma unroll
        for (int j = 0; j < SH::ITEMS; ++j)
            if (item_live[j]) *reinterpret_cast<u32x4*>(buf + item_dst[j]) = pre[j];
        __syncthreads();
        if (slab + 1 < nslabs) fetch(slab + 1);
#pragma unroll
        for (int ks = 0; ks < kSlabK / 32; ++ks) {
            if (ks % SH::KSPLIT != kp % SH::KSPLIT) continue;      // wave-uniform
            u32x4 a[OCF];
#pragma unroll
            for (int f = 0; f < OCF; ++f)
                a[f] = *reinterpret_cast<const u32x4*>(buf + (TT * kTileM + f * kTileOC) * kSlabPitch + frag_off + ks * 64);
#pragma unroll
            for (int u = 0; u < SH::TPW; ++u) {
                const int t = tg * SH::TPW + u;
                const u32x4 b = *reinterpret_cast<const u32x4*>(buf + t * kTileM * kSlabPitch + frag_off + ks * 64);
#pragma unroll
                for (int f = 0; f < OCF; ++f) acc[f][u] = mfma16<XT>(a[f], b, acc[f][u]);
            }
        }
        if (!DB) __syncthreads();
    }
    if (DB) __syncthreads();

    // Accumulators -> LDS as [K part][t][m][PITCH]; D[i = oc][j = m]: lane holds column j = lane % 16, rows 4 (lane / 16) + r.
    float* partial = reinterpret_cast<float*>(staged_lds);
    constexpr int SLAB_F = kTileM * SH::PITCH;
#pragma unroll
    for (int u = 0; u < SH::TPW; ++u)
#pragma unroll
        for (int f = 0; f < OCF; ++f)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                partial[(kp * TT + tg * SH::TPW + u) * SLAB_F + (lane & 15) * SH::PITCH + f * kTileOC + (lane >> 4) * 4 + r] = acc[f][u][r];
    __syncthreads();

    for (int e = tid; e < OUTS; e += NT) {
        const int slot = (e / TILE_OC) * SH::PITCH + e % TILE_OC;
        const int m = m0 + e / TILE_OC;
        const int oc = oc0 + e % TILE_OC;
        if (m >= g.M || oc >= g.Fout) continue;
        const float bv = bias != nullptr ? to_float(bias[oc]) : 0.0f;
        const int64_t o = static_cast<int64_t>(m) * g.Fout + oc;
        float v = v_init != nullptr ? to_float(v_init[o]) : 0.0f;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            if (t >= g.T) break;
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < SH::KSPLIT; ++w) sum += partial[(w * TT + t) * SLAB_F + slot];
            const float cur = sum + bv;
            spikes[t * g.spike_step_stride + o] = spike_value<XT>(lif_step(cur, v, lif));
        }
        v_out[o] = from_float<VT>(v);
    }
}

template <typename XT, typename VT, int TT, int OCF, bool DB>
int launch_staged_db(dim3 grid, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
                     void* v_out, const LifParams& lif, hipStream_t stream) {
    using SH = StagedShape<TT, OCF>;
    constexpr size_t lds = DB ? 2 * SH::slab_bytes : SH::lds_bytes;
    static_assert(lds <= 160 * 1024 && SH::acc_bytes <= lds, "slabs exceed LDS");
    auto kernel = linear_lif_staged_kernel<XT, VT, TT, OCF, DB>;
    if (lds > 64 * 1024) {
        static const hipError_t raised = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (raised != hipSuccess) return fail(SNNF_ERR_LAUNCH, "snnf_linear_lif: cannot reserve %zu bytes of LDS", lds);
    }
    kernel<<<grid, kStagedWaves * 64, lds, stream>>>(xs, g, static_cast<const XT*>(W), static_cast<const XT*>(bias),
                                                     static_cast<const VT*>(v_init), static_cast<XT*>(spikes),
                                                     static_cast<VT*>(v_out), lif);
    return check_launch("snnf_linear_lif");
}

template <typename XT, typename VT, int TT, int OCF>
int launch_staged(const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
                  void* v_out, const LifParams& lif, hipStream_t stream) {
    using SH = StagedShape<TT, OCF>;
    const dim3 grid((g.Fout + OCF * kTileOC - 1) / (OCF * kTileOC), (g.M + kTileM - 1) / kTileM);
    if (grid.y > 65535) return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: M=%d too large", g.M);
    // Two slab buffers where a CU gets one workgroup anyway (they would cost occupancy otherwise) and both fit LDS.
    constexpr bool can_double = 2 * SH::slab_bytes <= 160 * 1024;
    if constexpr (can_double) {
        if (static_cast<int64_t>(grid.x) * grid.y <= compute_units())
            return launch_staged_db<XT, VT, TT, OCF, true>(grid, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    }
    return launch_staged_db<XT, VT, TT, OCF, false>(grid, xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

template <typename XT, typename VT, bool FAST>
int launch_tt(const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
              void* v_out, const LifParams& lif, hipStream_t stream) {
    // Two feature fragments per workgroup (half the activation traffic) when that still leaves at least 128 workgroups.
    const bool wide = g.Fout % (2 * kTileOC) == 0 &&
                      static_cast<int64_t>(g.Fout / (2 * kTileOC)) * ((g.M + kTileM - 1) / kTileM) >= 128;
    if constexpr (FAST) {
        if (g.T > 2) {
            if (wide) {
                if (g.T <= 4) return launch_staged<XT, VT, 4, 2>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
                if (g.T <= 8) return launch_staged<XT, VT, 8, 2>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
                return launch_staged<XT, VT, 16, 2>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
            }
            if (g.T <= 4) return launch_staged<XT, VT, 4, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
            if (g.T <= 8) return launch_staged<XT, VT, 8, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
            return launch_staged<XT, VT, 16, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
        }
    }
    if (g.T <= 1) return launch_one<XT, VT, 1, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 2) return launch_one<XT, VT, 2, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 4) return launch_one<XT, VT, 4, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    if (g.T <= 8) return launch_one<XT, VT, 8, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
    return launch_one<XT, VT, 16, FAST, 1>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

template <typename XT, typename VT>
int launch(bool fast, const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init,
           void* spikes, void* v_out, const LifParams& lif, hipStream_t stream) {
    return fast ? launch_tt<XT, VT, true>(xs, g, W, bias, v_init, spikes, v_out, lif, stream)
                : launch_tt<XT, VT, false>(xs, g, W, bias, v_init, spikes, v_out, lif, stream);
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_linear_lif(const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                               const void* weight, const void* bias, int Fout, int w_dtype, const void* v_init,
                               int v_dtype, void* spikes, int64_t spike_step_stride, void* v_out, float v_threshold,
                               float v_reset, float tau, void* stream) {
    using namespace snnf;
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
        const void* vi = t0 == 0 ? v_init : v_out;
        void* sp = static_cast<char*>(spikes) + static_cast<int64_t>(t0) * spike_step_stride * xsize;
        int rc;
        if (x_dtype == SNNF_F32) rc = launch<float, float>(fast, ptrs, g, weight, bias, vi, sp, v_out, lif, hs);
        else if (x_dtype == SNNF_BF16)
            rc = v_dtype == SNNF_F32 ? launch<bf16_t, float>(fast, ptrs, g, weight, bias, vi, sp, v_out, lif, hs)
                                     : launch<bf16_t, bf16_t>(fast, ptrs, g, weight, bias, vi, sp, v_out, lif, hs);
        else
            rc = v_dtype == SNNF_F32 ? launch<f16_t, float>(fast, ptrs, g, weight, bias, vi, sp, v_out, lif, hs)
                                     : launch<f16_t, f16_t>(fast, ptrs, g, weight, bias, vi, sp, v_out, lif, hs);
        if (rc != SNNF_OK) return rc;
    }
    return SNNF_OK;
}
