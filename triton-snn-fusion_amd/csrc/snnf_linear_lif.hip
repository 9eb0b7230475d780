// Temporal Linear + LIF on the matrix cores: out^T[Fout, T*M] = W[Fout, Fin] . x^T, LIF recurrence in the epilogue.
//
// Both operands are K-contiguous in memory (x rows and W rows), which is exactly the per-lane operand order of
// v_mfma_f32_16x16x32 (8 consecutive k per lane), so fragments are loaded straight from global memory into registers.
// All T timesteps of a row tile share one weight fragment load (the weight is streamed once per workgroup, not once per
// timestep). The 8 (or, beyond 8 timesteps, 4) waves of a workgroup split K and prefetch their next K step while the
// current one multiplies; partial sums meet in LDS, then each thread runs the LIF recurrence over T for its (row, output
// feature) pair with the membrane in a register.
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

// Loads k .. k+7 of `row`; elements at or beyond `kmax` read as zero. FAST requires 16-byte aligned rows.
template <typename XT, bool FAST>
__device__ __forceinline__ u32x4 load_octet(const XT* __restrict__ row, int k, int kmax) {
    u32x4 out = {0u, 0u, 0u, 0u};
    if constexpr (sizeof(XT) == 2) {
        if (FAST && k + 8 <= kmax) {
            out = *reinterpret_cast<const u32x4*>(row + k);
        } else {
            const uint16_t* p = reinterpret_cast<const uint16_t*>(row);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo = (k + 2 * j) < kmax ? p[k + 2 * j] : 0u;
                const uint32_t hi = (k + 2 * j + 1) < kmax ? p[k + 2 * j + 1] : 0u;
                out[j] = lo | (hi << 16);
            }
        }
    } else {
        if (FAST && k + 8 <= kmax) {
            const f32x4 a = *reinterpret_cast<const f32x4*>(row + k);
            const f32x4 b = *reinterpret_cast<const f32x4*>(row + k + 4);
            out[0] = pack_bf16x2(a[0], a[1]);
            out[1] = pack_bf16x2(a[2], a[3]);
            out[2] = pack_bf16x2(b[0], b[1]);
            out[3] = pack_bf16x2(b[2], b[3]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = (k + 2 * j) < kmax ? to_float(row[k + 2 * j]) : 0.0f;
                const float hi = (k + 2 * j + 1) < kmax ? to_float(row[k + 2 * j + 1]) : 0.0f;
                out[j] = pack_bf16x2(lo, hi);
            }
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

// Waves per workgroup: they split K, so more waves mean more loads in flight per CU; their partial sums (1 KiB per wave
// and timestep) must fit the 64 KiB of static LDS.
template <int TT> struct LinWaves { static constexpr int value = TT <= 8 ? 8 : 4; };

template <typename XT, typename VT, int TT, bool FAST>
__global__ __launch_bounds__(LinWaves<TT>::value * 64) void linear_lif_kernel(StepPtrs xs, LinGeom g, const XT* __restrict__ W,
                                                                              const XT* __restrict__ bias,
                                                                              const VT* __restrict__ v_init, XT* __restrict__ spikes,
                                                                              VT* __restrict__ v_out, LifParams lif) {
    constexpr int NW = LinWaves<TT>::value;
    __shared__ float partial[NW][TT][kTileOC * kTileM];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int oc0 = blockIdx.x * kTileOC;
    const int m0 = blockIdx.y * kTileM;

    // Operand rows of this lane (clamped: out-of-range rows compute garbage that is never stored).
    const int a_row = min(oc0 + (lane & 15), g.Fout - 1);
    const int b_row = min(m0 + (lane & 15), g.M - 1);
    const int koff = (lane >> 4) * 8;
    const XT* __restrict__ wrow = W + static_cast<int64_t>(a_row) * g.Fin;
    const XT* xrow[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) xrow[t] = static_cast<const XT*>(xs.p[t]) + static_cast<int64_t>(b_row) * g.x_row_stride;

    f32x4 acc[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // K step s (32 elements of K) belongs to wave s % NW. Two register sets: the loads of a wave's next step are in flight
    // while the matrix instructions of the current one run.
    u32x4 a0, a1, b0[TT], b1[TT];
    auto fetch = [&](int s, u32x4& a, u32x4 (&b)[TT]) __attribute__((always_inline)) {
        const int k = s * 32 + koff;
        a = load_octet<XT, FAST>(wrow, k, g.Fin);
#pragma unroll
        for (int t = 0; t < TT; ++t) b[t] = load_octet<XT, FAST>(xrow[t], k, g.Fin);
    };
    auto multiply = [&](const u32x4& a, const u32x4 (&b)[TT]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[t] = mfma16<XT>(a, b[t], acc[t]);
    };
    int s = wave;
    if (s < g.ksteps) fetch(s, a0, b0);
    for (; s < g.ksteps; s += 2 * NW) {
        const bool more1 = s + NW < g.ksteps;
        if (more1) fetch(s + NW, a1, b1);
        multiply(a0, b0);
        if (s + 2 * NW < g.ksteps) fetch(s + 2 * NW, a0, b0);
        if (more1) multiply(a1, b1);
    }

    // D[i = oc][j = m]: lane holds column j = lane % 16, rows i = 4 * (lane / 16) + r.
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][(lane & 15) * kTileOC + (lane >> 4) * 4 + r] = acc[t][r];
    __syncthreads();

    // Thread e < 256 owns (row m_local = e / 16, feature oc_local = e % 16): consecutive threads write consecutive
    // features. The partial sums are added in a fixed order.
    const int e = threadIdx.x;
    if (e >= kTileOC * kTileM) return;
    const int m = m0 + (e >> 4);
    const int oc = oc0 + (e & 15);
    if (m >= g.M || oc >= g.Fout) return;
    const float bv = bias != nullptr ? to_float(bias[oc]) : 0.0f;
    const int64_t o = static_cast<int64_t>(m) * g.Fout + oc;
    float v = v_init != nullptr ? to_float(v_init[o]) : 0.0f;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
        if (t >= g.T) break;
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; w += 2) sum += partial[w][t][e] + partial[w + 1][t][e];
        const float cur = sum + bv;
        spikes[t * g.spike_step_stride + o] = spike_value<XT>(lif_step(cur, v, lif));
    }
    v_out[o] = from_float<VT>(v);
}

template <typename XT, typename VT, bool FAST>
int launch_tt(const StepPtrs& xs, const LinGeom& g, const void* W, const void* bias, const void* v_init, void* spikes,
              void* v_out, const LifParams& lif, hipStream_t stream) {
    const dim3 grid((g.Fout + kTileOC - 1) / kTileOC, (g.M + kTileM - 1) / kTileM);
    if (grid.y > 65535) return fail(SNNF_ERR_UNSUPPORTED, "snnf_linear_lif: M=%d too large", g.M);
    const XT* w = static_cast<const XT*>(W);
    const XT* b = static_cast<const XT*>(bias);
    const VT* vi = static_cast<const VT*>(v_init);
    XT* sp = static_cast<XT*>(spikes);
    VT* vo = static_cast<VT*>(v_out);
    if (g.T <= 1) linear_lif_kernel<XT, VT, 1, FAST><<<grid, LinWaves<1>::value * 64, 0, stream>>>(xs, g, w, b, vi, sp, vo, lif);
    else if (g.T <= 2) linear_lif_kernel<XT, VT, 2, FAST><<<grid, LinWaves<2>::value * 64, 0, stream>>>(xs, g, w, b, vi, sp, vo, lif);
    else if (g.T <= 4) linear_lif_kernel<XT, VT, 4, FAST><<<grid, LinWaves<4>::value * 64, 0, stream>>>(xs, g, w, b, vi, sp, vo, lif);
    else if (g.T <= 8) linear_lif_kernel<XT, VT, 8, FAST><<<grid, LinWaves<8>::value * 64, 0, stream>>>(xs, g, w, b, vi, sp, vo, lif);
    else linear_lif_kernel<XT, VT, 16, FAST><<<grid, LinWaves<16>::value * 64, 0, stream>>>(xs, g, w, b, vi, sp, vo, lif);
    return check_launch("snnf_linear_lif");
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
        bool fast = Fin % per16 == 0 && x_row_stride % per16 == 0 && aligned_to(weight, 16);
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
