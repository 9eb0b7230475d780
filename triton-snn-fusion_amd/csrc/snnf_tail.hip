// LIF -> global average pool -> Linear, summed over T (the classifier tail of a spiking network).
//
//   out_sum[n, k] = sum_t ( W[k, :] . mean_hw(s_t[n, :, :, :]) + b[k] ) = (W[k, :] . count[n, :]) / HW + T * b[k]
//
// where count[n, c] is the number of spikes of plane (n, c) over all T steps: the pooled activations are never
// materialised per step. Launch 1 streams x once (HBM-bound, 16-byte accesses where the operands allow), keeps the membrane
// in registers, counts spikes per plane in LDS and writes the integer counts to the workspace; launch 2 is a small GEMV
// over the counts: wave-shuffle reductions for a few samples or classes, the matrix cores for batches.
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "snnf_common.h"

namespace snnf {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 4;        // neurons per thread in the pooling kernel
constexpr int kMaxPlanes = 1024;  // planes per workgroup (HW == 1 gives kThreads * kItems planes)

template <typename XT, typename VT>
__global__ __launch_bounds__(kThreads) void lif_pool_kernel(StepPtrs xs, int T, int planes, int HW, int planes_per_block,
                                                            const VT* __restrict__ v_init, VT* __restrict__ v_out,
                                                            int* __restrict__ counts, LifParams lif) {
    __shared__ int plane_count[kMaxPlanes];
    const int plane0 = blockIdx.x * planes_per_block;
    const int planes_here = min(planes_per_block, planes - plane0);
    const int elems = planes_here * HW;
    const int64_t base = static_cast<int64_t>(plane0) * HW;
    for (int i = threadIdx.x; i < planes_here; i += kThreads) plane_count[i] = 0;
    __syncthreads();

    // Chunks of kThreads * kItems neurons: one chunk unless a single plane is larger than that.
    for (int c0 = 0; c0 < elems; c0 += kThreads * kItems) {
        float v[kItems];
        int plane_of[kItems];
        int fired_total[kItems];
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            const int i = c0 + threadIdx.x + k * kThreads;
            plane_of[k] = i < elems ? i / HW : -1;
            fired_total[k] = 0;
            v[k] = (i < elems && v_init != nullptr) ? to_float(v_init[base + i]) : 0.0f;
        }
        for (int t = 0; t < T; ++t) {
            const XT* __restrict__ x = static_cast<const XT*>(xs.p[t]) + base;
#pragma unroll
            for (int k = 0; k < kItems; ++k) {
                const int i = c0 + threadIdx.x + k * kThreads;
                if (i < elems) fired_total[k] += lif_step(to_float(x[i]), v[k], lif) ? 1 : 0;
            }
        }
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            const int i = c0 + threadIdx.x + k * kThreads;
            // Wave-level reduction when the whole wave sits in one plane, LDS atomics otherwise.
            const int my_plane = plane_of[k];
            const int lead_plane = __shfl(my_plane, 0);
            if (__all(my_plane == lead_plane)) {
                int sum = fired_total[k];
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
                if ((threadIdx.x & 63) == 0 && lead_plane >= 0) atomicAdd(&plane_count[lead_plane], sum);
            } else if (my_plane >= 0 && fired_total[k] != 0) {
                atomicAdd(&plane_count[my_plane], fired_total[k]);
            }
            if (i < elems) v_out[base + i] = from_float<VT>(v[k]);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < planes_here; i += kThreads) counts[plane0 + i] = plane_count[i];
}

// Vector variant of the pooling kernel: a thread owns 8 consecutive neurons of the workgroup's planes per pass, fetched
// with 16-byte loads, four timesteps in flight at a time; a thread's spikes are merged per plane before they reach the
// LDS counters. The host guarantees that a workgroup's first neuron is a multiple of 8 and that all bases are 16-byte
// aligned; only the last 8 neurons of the last workgroup may be ragged and are moved one by one.
constexpr int kVec = 8;

template <typename XT, typename VT, int TC>
__global__ __launch_bounds__(kThreads) void lif_pool_vec_kernel(StepPtrs xs, int T, int planes, int HW, int planes_per_block,
                                                                const VT* __restrict__ v_init, VT* __restrict__ v_out,
                                                                int* __restrict__ counts, LifParams lif, int stream_out) {
    __shared__ int plane_count[kMaxPlanes];
    const int plane0 = blockIdx.x * planes_per_block;
    const int planes_here = min(planes_per_block, planes - plane0);
    const int elems = planes_here * HW;
    const int64_t base = static_cast<int64_t>(plane0) * HW;
    for (int i = threadIdx.x; i < planes_here; i += kThreads) plane_count[i] = 0;
    __syncthreads();

    // A workgroup whose neuron count is a multiple of 8 (all but, at most, the last one) moves whole vectors only; its
    // loop body has no branch around a load, so all loads of a pass are in flight together.
    auto pass = [&](int i0, auto whole_tag) __attribute__((always_inline)) {
        constexpr bool whole = decltype(whole_tag)::value;
        float v[kVec];
        int fired[kVec];
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
            v[j] = 0.0f;
            fired[j] = 0;
        }
        if (v_init != nullptr) {
            if constexpr (whole) {
                const Pack<VT, kVec> pv = *reinterpret_cast<const Pack<VT, kVec>*>(v_init + base + i0);
#pragma unroll
                for (int j = 0; j < kVec; ++j) v[j] = to_float(pv.v[j]);
            } else {
#pragma unroll
                for (int j = 0; j < kVec; ++j)
                    if (i0 + j < elems) v[j] = to_float(v_init[base + i0 + j]);
            }
        }
        if constexpr (whole && TC > 0) {
            // T == TC known at compile time: every timestep's load is issued before the recurrence starts. (Fetching
            // the next pass ahead as well measured no faster.)
            Pack<XT, kVec> px[TC > 0 ? TC : 1];
#pragma unroll
            for (int t = 0; t < TC; ++t) px[t] = *reinterpret_cast<const Pack<XT, kVec>*>(static_cast<const XT*>(xs.p[t]) + base + i0);
#pragma unroll
            for (int t = 0; t < TC; ++t)
#pragma unroll
                for (int j = 0; j < kVec; ++j) fired[j] += lif_step(to_float(px[t].v[j]), v[j], lif) ? 1 : 0;
        } else {
            for (int t0 = 0; t0 < T; t0 += 4) {
                Pack<XT, kVec> px[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (t0 + u < T) {
                        const XT* __restrict__ x = static_cast<const XT*>(xs.p[t0 + u]) + base + i0;
                        if constexpr (whole) {
                            px[u] = *reinterpret_cast<const Pack<XT, kVec>*>(x);
                        } else {
#pragma unroll
                            for (int j = 0; j < kVec; ++j) px[u].v[j] = i0 + j < elems ? x[j] : XT{};
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (t0 + u < T) {
#pragma unroll
                        for (int j = 0; j < kVec; ++j) fired[j] += lif_step(to_float(px[u].v[j]), v[j], lif) ? 1 : 0;
                    }
                }
            }
        }
        if constexpr (whole) {
            Pack<VT, kVec> pv;
#pragma unroll
            for (int j = 0; j < kVec; ++j) pv.v[j] = from_float<VT>(v[j]);
            if (stream_out) store_streaming(v_out + base + i0, pv);
            else *reinterpret_cast<Pack<VT, kVec>*>(v_out + base + i0) = pv;
        } else {
#pragma unroll
            for (int j = 0; j < kVec; ++j)
                if (i0 + j < elems) v_out[base + i0 + j] = from_float<VT>(v[j]);
        }
        // Spikes of consecutive neurons of one plane are summed before they go to that plane's counter; a wave whose
        // neurons all lie in one plane adds them up with shuffles first (one LDS atomic per wave instead of 64 on the
        // same address).
        int p = i0 / HW;
        int rem = i0 - p * HW;
        const bool one_plane = rem + kVec <= HW && whole;      // this thread's 8 neurons lie inside plane p
        const int lead = __shfl(p, 0);
        const bool full_wave = __builtin_amdgcn_ballot_w64(true) == ~0ull;   // the shuffles below need all 64 lanes
        if (full_wave && __all(one_plane && p == lead)) {
            int sum = 0;
#pragma unroll
            for (int j = 0; j < kVec; ++j) sum += fired[j];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
            if ((threadIdx.x & 63) == 0 && sum != 0) atomicAdd(&plane_count[lead], sum);
        } else {
            int run = 0;
#pragma unroll
            for (int j = 0; j < kVec; ++j) {
                if (i0 + j < elems) {
                    run += fired[j];
                    if (++rem == HW) {
                        if (run != 0) atomicAdd(&plane_count[p], run);
                        run = 0;
                        rem = 0;
                        ++p;
                    }
                }
            }
            if (run != 0) atomicAdd(&plane_count[p], run);
        }
    };
    if (elems % kVec == 0) {
        for (int i0 = threadIdx.x * kVec; i0 < elems; i0 += kThreads * kVec) pass(i0, std::true_type{});
    } else {
        for (int i0 = threadIdx.x * kVec; i0 < elems; i0 += kThreads * kVec) pass(i0, std::false_type{});
    }
    __syncthreads();
    for (int i = threadIdx.x; i < planes_here; i += kThreads) counts[plane0 + i] = plane_count[i];
}

// One workgroup: one sample n, kWavesPerBlock * kRowsPerWave output rows; the sample's spike counts sit in LDS.
constexpr int kRowsPerWave = 4;

template <typename XT>
__global__ __launch_bounds__(kThreads) void count_linear_kernel(const int* __restrict__ counts, int C, int K,
                                                                const XT* __restrict__ W, const XT* __restrict__ bias,
                                                                XT* __restrict__ out, float inv_hw, float steps) {
    extern __shared__ float cnt[];
    const int n = blockIdx.y;
    for (int c = threadIdx.x; c < C; c += kThreads) cnt[c] = static_cast<float>(counts[n * C + c]);
    __syncthreads();
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int k0 = (blockIdx.x * (kThreads / 64) + wave) * kRowsPerWave;
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int k = k0 + r;
        if (k >= K) break;
        const XT* __restrict__ row = W + static_cast<int64_t>(k) * C;
        float acc = 0.0f;
        for (int c = lane; c < C; c += 64) acc = fmaf(to_float(row[c]), cnt[c], acc);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
        if (lane == 0) {
            float o = acc * inv_hw;
            if (bias != nullptr) o += steps * to_float(bias[k]);
            out[static_cast<int64_t>(n) * K + k] = from_float<XT>(o);
        }
    }
}

// Vector variant (C a multiple of 8, 16-byte aligned weight): no LDS and no barrier; a lane fetches 8 consecutive weights
// of each of its wave's kRowsPerWave rows with 16-byte loads, all rows in flight together, and the 8 matching counts of
// kSamplesPerWave samples (1: sharing a weight vector among 4 samples saved 2 % at 64 samples x 1000 classes and cost
// 15-20 % at the sizes of the network tails, where the shuffle reductions of a wave then run one after the other).
constexpr int kSamplesPerWave = 1;

template <typename XT>
__global__ __launch_bounds__(kThreads) void count_linear_vec_kernel(const int* __restrict__ counts, int N, int C, int K,
                                                                    const XT* __restrict__ W, const XT* __restrict__ bias,
                                                                    XT* __restrict__ out, float inv_hw, float steps) {
    const int n0 = blockIdx.y * kSamplesPerWave;
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int k0 = (blockIdx.x * (kThreads / 64) + wave) * kRowsPerWave;
    if (k0 >= K) return;
    float acc[kRowsPerWave][kSamplesPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
        for (int i = 0; i < kSamplesPerWave; ++i) acc[r][i] = 0.0f;
    for (int c0 = lane * kVec; c0 < C; c0 += 64 * kVec) {
        Pack<int, kVec> pc[kSamplesPerWave];
#pragma unroll
        for (int i = 0; i < kSamplesPerWave; ++i) {
            const int n = min(n0 + i, N - 1);   // samples beyond N re-read the last one and are not stored
            pc[i] = *reinterpret_cast<const Pack<int, kVec>*>(counts + static_cast<int64_t>(n) * C + c0);
        }
        Pack<XT, kVec> pw[kRowsPerWave];
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) {
            const int k = min(k0 + r, K - 1);   // rows beyond K re-read the last one and are not stored
            pw[r] = *reinterpret_cast<const Pack<XT, kVec>*>(W + static_cast<int64_t>(k) * C + c0);
        }
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
            for (int j = 0; j < kVec; ++j) {
                const float w = to_float(pw[r].v[j]);
#pragma unroll
                for (int i = 0; i < kSamplesPerWave; ++i) acc[r][i] = fmaf(w, static_cast<float>(pc[i].v[j]), acc[r][i]);
            }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
        for (int i = 0; i < kSamplesPerWave; ++i) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) acc[r][i] += __shfl_xor(acc[r][i], off);
        }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) {
            const int k = k0 + r;
            if (k >= K) continue;
            const float bv = bias != nullptr ? steps * to_float(bias[k]) : 0.0f;
#pragma unroll
            for (int i = 0; i < kSamplesPerWave; ++i) {
                const int n = n0 + i;
                if (n < N) out[static_cast<int64_t>(n) * K + k] = from_float<XT>(acc[r][i] * inv_hw + bv);
            }
        }
    }
}

// Matrix-core variant for batches of samples (16-bit weights, C a multiple of 32, counts below 65536): a workgroup owns 16
// classes x 16 samples; its 4 waves deal the steps of 32 channels among themselves and meet in LDS, summed in wave order.
// A count is exact in neither 16-bit format, so it enters as two exact operands, count & 255 and count >> 8, against the
// same weight fragment: out = (W . low + 256 * (W . high)) / HW + T * b with fp32 accumulation.
typedef __bf16 tail_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 tail_f16x8 __attribute__((ext_vector_type(8)));
typedef float tail_f32x4 __attribute__((ext_vector_type(4)));
constexpr int kMmTile = 16;
constexpr int kMmMaxCount = 65535;
constexpr int kMmMinSamples = 8;   // below 8 samples or 64 classes the tile is mostly padding: the shuffle kernel is quicker
constexpr int kMmMinClasses = 64;

template <typename XT>
__device__ __forceinline__ tail_f32x4 tail_mfma(snnf_u32x4 a, snnf_u32x4 b, tail_f32x4 c) {
    if constexpr (dtype_of<XT>::value == SNNF_F16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(tail_f16x8, a), __builtin_bit_cast(tail_f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(tail_bf16x8, a), __builtin_bit_cast(tail_bf16x8, b), c, 0, 0, 0);
    }
}

// Two integers below 256 as a pair of 16-bit floats (exact in both formats).
template <typename XT>
__device__ __forceinline__ uint32_t small_pair(int a, int b) {
    if constexpr (dtype_of<XT>::value == SNNF_F16) {
        return float_to_f16_bits(static_cast<float>(a)) | (float_to_f16_bits(static_cast<float>(b)) << 16);
    } else {
        return (__float_as_uint(static_cast<float>(a)) >> 16) | (__float_as_uint(static_cast<float>(b)) & 0xffff0000u);
    }
}

template <typename XT>
__global__ __launch_bounds__(kThreads) void count_linear_mm_kernel(const int* __restrict__ counts, int N, int C, int K,
                                                                   const XT* __restrict__ W, const XT* __restrict__ bias,
                                                                   XT* __restrict__ out, float inv_hw, float steps) {
    static_assert(sizeof(XT) == 2, "16-bit weights");
    __shared__ float part[kThreads / 64][64 * 4];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int k0 = blockIdx.x * kMmTile;
    const int n0 = blockIdx.y * kMmTile;
    // Operand order of v_mfma_f32_16x16x32: lane l holds 8 consecutive channels, 8 * (l / 16) on, of row l % 16.
    const int row = lane & 15;
    const int sub = (lane >> 4) * 8;
    const XT* __restrict__ w_row = W + static_cast<int64_t>(min(k0 + row, K - 1)) * C + sub;         // rows beyond K: re-read, not stored
    const int* __restrict__ c_row = counts + static_cast<int64_t>(min(n0 + row, N - 1)) * C + sub;   // samples beyond N likewise
    tail_f32x4 acc_lo = {0.0f, 0.0f, 0.0f, 0.0f};
    tail_f32x4 acc_hi = {0.0f, 0.0f, 0.0f, 0.0f};
    const int ksteps = C >> 5;
    for (int ks = wave; ks < ksteps; ks += kThreads / 64) {
        const snnf_u32x4 wf = *reinterpret_cast<const snnf_u32x4*>(w_row + ks * 32);
        const Pack<int, 4> c0 = *reinterpret_cast<const Pack<int, 4>*>(c_row + ks * 32);
        const Pack<int, 4> c1 = *reinterpret_cast<const Pack<int, 4>*>(c_row + ks * 32 + 4);
        snnf_u32x4 lo, hi;
        lo[0] = small_pair<XT>(c0.v[0] & 255, c0.v[1] & 255);
        lo[1] = small_pair<XT>(c0.v[2] & 255, c0.v[3] & 255);
        lo[2] = small_pair<XT>(c1.v[0] & 255, c1.v[1] & 255);
        lo[3] = small_pair<XT>(c1.v[2] & 255, c1.v[3] & 255);
        hi[0] = small_pair<XT>(c0.v[0] >> 8, c0.v[1] >> 8);
        hi[1] = small_pair<XT>(c0.v[2] >> 8, c0.v[3] >> 8);
        hi[2] = small_pair<XT>(c1.v[0] >> 8, c1.v[1] >> 8);
        hi[3] = small_pair<XT>(c1.v[2] >> 8, c1.v[3] >> 8);
        acc_lo = tail_mfma<XT>(wf, lo, acc_lo);
        acc_hi = tail_mfma<XT>(wf, hi, acc_hi);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) part[wave][lane * 4 + j] = fmaf(256.0f, acc_hi[j], acc_lo[j]);
    __syncthreads();
    // Thread t finishes output t of the tile: class 4 * (l / 16) + j of sample l % 16, with l = t / 4 and j = t % 4.
    float sum = part[0][threadIdx.x];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) sum += part[w][threadIdx.x];
    const int l = threadIdx.x >> 2;
    const int k = k0 + 4 * (l >> 4) + (threadIdx.x & 3);
    const int n = n0 + (l & 15);
    if (k < K && n < N) {
        const float bv = bias != nullptr ? steps * to_float(bias[k]) : 0.0f;
        out[static_cast<int64_t>(n) * K + k] = from_float<XT>(sum * inv_hw + bv);
    }
}

// The whole tail in one launch, for tails as small as those at the end of a network: a workgroup owns one sample and a range
// of classes. It runs the sample's LIF recurrence (a thread owns 8 consecutive neurons per pass, 16-byte loads, four timesteps
// in flight), counts the spikes per channel in LDS and multiplies its classes' weight rows with the counts right away: no
// counts in memory, no second launch. The workgroups of a sample that differ in their class range repeat the recurrence (the
// sample's activations come from L2 then); the first of them writes the membrane. The products run like
// count_linear_vec_kernel's (a wave owns kRowsPerWave rows, a lane 8 consecutive channels per trip, shuffle reduction), so the
// two paths give the same sums bit for bit.
constexpr int kOneMaxC = 2048;                    // channels of a sample whose counters fit the workgroup's LDS array
constexpr int64_t kOneMaxSampleWork = 32 * 1024;  // T * C * HW of one sample, at most: 128 LIF steps per thread (larger samples are
                                                  // better spread over many workgroups by the pooling kernel of the two-launch path)

// out[n, k] = (Wt[k, :] . counts / HW + steps * bias[k]) * out_scale for the classes of this workgroup's range, from the
// per-channel spike counts of sample n in LDS: kRowsPerWave rows per wave and pass, a lane takes 8 channels at a time.
template <typename XT>
__device__ __forceinline__ void classify_counts(const int* plane_count, int n, int C, int K, int classes_per_block, const XT* __restrict__ Wt,
                                                const XT* __restrict__ bias, XT* __restrict__ out, float inv_hw, float steps, float out_scale) {
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int k_begin = blockIdx.x * classes_per_block;
    const int k_end = min(K, k_begin + classes_per_block);
    for (int k0 = k_begin + wave * kRowsPerWave; k0 < k_end; k0 += (kThreads / 64) * kRowsPerWave) {
        float acc[kRowsPerWave];
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) acc[r] = 0.0f;
        for (int c0 = lane * kVec; c0 < C; c0 += 64 * kVec) {
            const Pack<int, kVec> pc = *reinterpret_cast<const Pack<int, kVec>*>(plane_count + c0);
            Pack<XT, kVec> pw[kRowsPerWave];
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r) {
                const int k = min(k0 + r, K - 1);   // rows beyond the range re-read the last one and are not stored
                pw[r] = *reinterpret_cast<const Pack<XT, kVec>*>(Wt + static_cast<int64_t>(k) * C + c0);
            }
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
                for (int j = 0; j < kVec; ++j) acc[r] = fmaf(to_float(pw[r].v[j]), static_cast<float>(pc.v[j]), acc[r]);
        }
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) acc[r] += __shfl_xor(acc[r], off);
        }
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r) {
                const int k = k0 + r;
                if (k >= k_end) continue;
                const float bv = bias != nullptr ? steps * to_float(bias[k]) : 0.0f;
                const float sum = acc[r] * inv_hw + bv;
                out[static_cast<int64_t>(n) * K + k] = from_float<XT>(out_scale == 1.0f ? sum : sum * out_scale);
            }
        }
    }
}

template <typename XT, typename VT>
__global__ __launch_bounds__(kThreads) void lif_pool_linear_one_kernel(StepPtrs xs, int T, int C, int HW, int K, int classes_per_block,
                                                                       const VT* __restrict__ v_init, VT* __restrict__ v_out,
                                                                       const XT* __restrict__ Wt, const XT* __restrict__ bias,
                                                                       XT* __restrict__ out, LifParams lif, float inv_hw, float steps) {
    __shared__ __align__(16) int plane_count[kOneMaxC];
    const int n = blockIdx.y;
    const int elems = C * HW;                                    // a multiple of 8 (host)
    const int64_t base = static_cast<int64_t>(n) * elems;
    const bool writes_v = blockIdx.x == 0;
    for (int i = threadIdx.x; i < C; i += kThreads) plane_count[i] = 0;
    __syncthreads();
    for (int i0 = threadIdx.x * kVec; i0 < elems; i0 += kThreads * kVec) {
        float v[kVec];
        int fired[kVec];
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
            v[j] = 0.0f;
            fired[j] = 0;
        }
        if (v_init != nullptr) {
            const Pack<VT, kVec> pv = *reinterpret_cast<const Pack<VT, kVec>*>(v_init + base + i0);
#pragma unroll
            for (int j = 0; j < kVec; ++j) v[j] = to_float(pv.v[j]);
        }
        for (int t0 = 0; t0 < T; t0 += 4) {
            Pack<XT, kVec> px[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (t0 + u < T) px[u] = *reinterpret_cast<const Pack<XT, kVec>*>(static_cast<const XT*>(xs.p[t0 + u]) + base + i0);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (t0 + u < T) {
#pragma unroll
                    for (int j = 0; j < kVec; ++j) fired[j] += lif_step(to_float(px[u].v[j]), v[j], lif) ? 1 : 0;
                }
            }
        }
        if (writes_v) {
            Pack<VT, kVec> pv;
#pragma unroll
            for (int j = 0; j < kVec; ++j) pv.v[j] = from_float<VT>(v[j]);
            *reinterpret_cast<Pack<VT, kVec>*>(v_out + base + i0) = pv;
        }
        // Spikes of consecutive neurons of one channel are summed before they go to that channel's counter.
        int p = i0 / HW;
        int rem = i0 - p * HW;
        int run = 0;
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
            run += fired[j];
            if (++rem == HW) {
                if (run != 0) atomicAdd(&plane_count[p], run);
                run = 0;
                rem = 0;
                ++p;
            }
        }
        if (run != 0) atomicAdd(&plane_count[p], run);
    }
    __syncthreads();
    classify_counts<XT>(plane_count, n, C, K, classes_per_block, Wt, bias, out, inv_hw, steps, 1.0f);
}

// Average pool and classifier on bit-packed spikes (one byte = 8 channels of a pixel), summed over T: the workgroup of a
// sample and a class range counts the sample's spikes per channel (a thread walks the bytes of one channel group and a
// share of its pixels, with one byte-wide counter per channel in two registers) and applies its weight rows.
constexpr int kSpikeStageBytes = 32 * 1024;   // a sample's bit-packed spikes of all timesteps, staged in LDS when they fit

template <typename XT, bool STAGED>
__global__ __launch_bounds__(kThreads) void spike_pool_linear_kernel(const unsigned char* __restrict__ spikes, int64_t step_stride, int T, int C8,
                                                                    int HW, int parts, int K, int classes_per_block,
                                                                    const XT* __restrict__ Wt, const XT* __restrict__ bias,
                                                                    XT* __restrict__ out, float inv_hw, float steps, float out_scale) {
    __shared__ __align__(16) int plane_count[kOneMaxC];
    __shared__ __align__(16) unsigned char staged[STAGED ? kSpikeStageBytes : 16];
    const int n = blockIdx.y;
    const int C = C8 * 8;
    for (int i = threadIdx.x; i < C; i += kThreads) plane_count[i] = 0;
    const int sample_bytes = C8 * HW;
    if constexpr (STAGED) {
        // The sample's bytes of every timestep are contiguous: coalesced 16-byte loads bring them into LDS (a multiple of 16
        // bytes at a 16-byte aligned address, checked on the host), and the counting below reads single bytes from there.
        const int vecs = sample_bytes / 16;
        for (int i = threadIdx.x; i < T * vecs; i += kThreads) {
            const int t = i / vecs;
            const int v = i - t * vecs;
            *reinterpret_cast<uint4*>(staged + t * sample_bytes + v * 16) =
                *reinterpret_cast<const uint4*>(spikes + static_cast<int64_t>(t) * step_stride + static_cast<int64_t>(n) * sample_bytes + v * 16);
        }
    }
    __syncthreads();
    const int per_part = (HW + parts - 1) / parts;
    for (int u = threadIdx.x; u < C8 * parts; u += kThreads) {
        const int c8 = u / parts;
        const int part = u - c8 * parts;
        const int p_begin = part * per_part, p_end = min(HW, p_begin + per_part);
        const int64_t base = (static_cast<int64_t>(n) * C8 + c8) * HW;
        uint32_t lo = 0, hi = 0;
        int pending = 0;
        auto flush = [&]() {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int a = static_cast<int>((lo >> (8 * j)) & 255u), b = static_cast<int>((hi >> (8 * j)) & 255u);
                if (a != 0) atomicAdd(&plane_count[c8 * 8 + j], a);
                if (b != 0) atomicAdd(&plane_count[c8 * 8 + 4 + j], b);
            }
            lo = hi = 0;
            pending = 0;
        };
        // 8 pixels x 4 timesteps per trip, all 32 loads in flight together (positions beyond the range re-read its last byte
        // and count as zero: no branch around a load).
        for (int p0 = p_begin; p0 < p_end; p0 += 8) {
            for (int t0 = 0; t0 < T; t0 += 4) {
                uint32_t byte[4][8];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if constexpr (STAGED) {
                        const unsigned char* src = staged + min(t0 + u, T - 1) * sample_bytes + c8 * HW;
#pragma unroll
                        for (int j = 0; j < 8; ++j) byte[u][j] = src[min(p0 + j, p_end - 1)];
                    } else {
                        const unsigned char* __restrict__ src = spikes + static_cast<int64_t>(min(t0 + u, T - 1)) * step_stride + base;
#pragma unroll
                        for (int j = 0; j < 8; ++j) byte[u][j] = src[min(p0 + j, p_end - 1)];
                    }
                }
                if (pending > 255 - 32) flush();
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t b = (t0 + u < T && p0 + j < p_end) ? byte[u][j] : 0u;
                        lo += __umul24(b & 15u, 0x00204081u) & 0x01010101u;
                        hi += __umul24(b >> 4, 0x00204081u) & 0x01010101u;
                    }
                pending += 32;
            }
        }
        flush();
    }
    __syncthreads();
    classify_counts<XT>(plane_count, n, C, K, classes_per_block, Wt, bias, out, inv_hw, steps, out_scale);
}

// Class ranges per sample of the one-launch tail: at least 16 classes each (one pass of the workgroup's four waves), no more
// workgroups than two per compute unit. 0: the shape takes the two launches.
int one_launch_class_blocks(int T, int N, int C, int HW, int K) {
    const int64_t work = static_cast<int64_t>(T) * C * HW;
    if (C > kOneMaxC || C % kVec != 0 || (static_cast<int64_t>(C) * HW) % kVec != 0 || work > kOneMaxSampleWork) return 0;
    const int rows_per_pass = (kThreads / 64) * kRowsPerWave;
    return std::max(1, std::min((K + rows_per_pass - 1) / rows_per_pass, 512 / std::max(1, N)));
}

template <typename XT, typename VT>
int run(const StepPtrs& xs, int T, int planes, int HW, const void* v_init, void* v_out, int* counts,
        const LifParams& lif, hipStream_t stream) {
    // Vector variant: about kThreads * kVec neurons per workgroup, whole planes, every workgroup starting at a multiple
    // of 8 neurons, all bases 16-byte aligned.
    bool aligned = aligned_to(v_out, 16) && (v_init == nullptr || aligned_to(v_init, 16));
    for (int t = 0; t < T; ++t) aligned = aligned && aligned_to(xs.p[t], 16);
    // Planes per workgroup: whole planes, a multiple of 8 neurons per workgroup, up to 4 passes of kThreads * kVec neurons,
    // chosen for the fewest idle lanes in the last pass (the first candidate wins unless a smaller one is 2 % better).
    const int pass_elems = kThreads * kVec;
    int vpb = 0;
    double best_eff = 0.0;
    // Several passes per workgroup only while that leaves 1024 workgroups or more.
    const int64_t one_pass = std::max<int64_t>(1, pass_elems / HW);
    const int64_t cand_max = std::min<int64_t>(std::max<int64_t>(1, (4 * pass_elems) / HW), std::max<int64_t>(one_pass, planes / 1024));
    for (int cand = static_cast<int>(std::min<int64_t>(kMaxPlanes, cand_max)); cand >= 1; --cand) {
        const int64_t e = static_cast<int64_t>(cand) * HW;
        if (cand < planes && e % kVec != 0) continue;
        const int64_t passes = (e + pass_elems - 1) / pass_elems;
        const double eff = static_cast<double>(e) / static_cast<double>(passes * pass_elems);
        if (eff > best_eff + 0.02) {
            best_eff = eff;
            vpb = cand;
        }
        if (cand >= planes) break;   // one workgroup holds everything: nothing smaller to consider
    }
    if (aligned && vpb > 0) {
        if (vpb > planes) vpb = planes;
        const int blocks = (planes + vpb - 1) / vpb;
        const VT* vi = static_cast<const VT*>(v_init);
        VT* vo = static_cast<VT*>(v_out);
        const int stream_out = static_cast<int64_t>(planes) * HW * static_cast<int64_t>(sizeof(VT)) >= kStreamOutBytes ? 1 : 0;   // see store_streaming
        if (T == 4) lif_pool_vec_kernel<XT, VT, 4><<<dim3(blocks), kThreads, 0, stream>>>(xs, T, planes, HW, vpb, vi, vo, counts, lif, stream_out);
        else if (T == 8) lif_pool_vec_kernel<XT, VT, 8><<<dim3(blocks), kThreads, 0, stream>>>(xs, T, planes, HW, vpb, vi, vo, counts, lif, stream_out);
        else lif_pool_vec_kernel<XT, VT, 0><<<dim3(blocks), kThreads, 0, stream>>>(xs, T, planes, HW, vpb, vi, vo, counts, lif, stream_out);
        return check_launch("snnf_lif_pool_linear(pool)");
    }
    int ppb = (kThreads * kItems) / HW;
    if (ppb < 1) ppb = 1;   // a plane larger than one chunk: the workgroup walks it chunk by chunk
    if (ppb > kMaxPlanes) ppb = kMaxPlanes;
    const int blocks = (planes + ppb - 1) / ppb;
    lif_pool_kernel<XT, VT><<<dim3(blocks), kThreads, 0, stream>>>(xs, T, planes, HW, ppb, static_cast<const VT*>(v_init),
                                                                  static_cast<VT*>(v_out), counts, lif);
    return check_launch("snnf_lif_pool_linear(pool)");
}

template <typename XT>
void run_linear(bool vec, bool matrix, dim3 grid, size_t lds, hipStream_t hs, const int* counts, int C, int K, const void* W,
                const void* bias, void* out, float inv_hw, float steps) {
    if constexpr (sizeof(XT) == 2) {
        if (matrix) {
            const int N = static_cast<int>(grid.y);
            const dim3 mgrid((K + kMmTile - 1) / kMmTile, (N + kMmTile - 1) / kMmTile);
            count_linear_mm_kernel<XT><<<mgrid, kThreads, 0, hs>>>(counts, N, C, K, static_cast<const XT*>(W),
                                                                  static_cast<const XT*>(bias), static_cast<XT*>(out), inv_hw, steps);
            return;
        }
    }
    if (vec) {
        const int N = static_cast<int>(grid.y);
        const dim3 vgrid(grid.x, (N + kSamplesPerWave - 1) / kSamplesPerWave);
        count_linear_vec_kernel<XT><<<vgrid, kThreads, 0, hs>>>(counts, N, C, K, static_cast<const XT*>(W), static_cast<const XT*>(bias),
                                                               static_cast<XT*>(out), inv_hw, steps);
    } else
        count_linear_kernel<XT><<<grid, kThreads, lds, hs>>>(counts, C, K, static_cast<const XT*>(W), static_cast<const XT*>(bias),
                                                            static_cast<XT*>(out), inv_hw, steps);
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_lif_pool_linear_launches(int T, int N, int C, int H, int W, int K) {
    if (T < 1 || N < 1 || C < 1 || H < 1 || W < 1 || K < 1) return 0;
    const int64_t hw = static_cast<int64_t>(H) * W;
    if (hw > (1 << 24)) return 2;
    return snnf::one_launch_class_blocks(T, N, C, static_cast<int>(hw), K) > 0 ? 1 : 2;
}

extern "C" size_t snnf_lif_pool_linear_workspace_bytes(int N, int C) {
    if (N < 1 || C < 1) return 0;
    return static_cast<size_t>(N) * static_cast<size_t>(C) * sizeof(int);
}

namespace snnf {
namespace {

// Shared body of the two entry points: `counts` is N * C ints of device memory (the caller's workspace or the library's
// own static array).
int lif_pool_linear_impl(const char* who, const void* const* xs, int T, int N, int C, int H, int W, int x_dtype,
                         const void* v_init, int v_dtype, const void* fc_weight, const void* fc_bias, int K,
                         int w_dtype, void* out_sum, void* v_out, int* counts,
                         float v_threshold, float v_reset, float tau, void* stream) {
    if (T > SNNF_MAX_T_PER_LAUNCH)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_temporal_length: T=%d exceeds %d", who, T, SNNF_MAX_T_PER_LAUNCH);
    if (!valid_dtype(x_dtype) || !valid_dtype(v_dtype) || !valid_dtype(w_dtype))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: unknown dtype code", who);
    if (w_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_dtype: fc_weight/fc_bias dtype must match x", who);
    if (v_dtype != SNNF_F32 && v_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_dtype: membrane dtype must be fp32 or the activation dtype", who);
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_tau: tau must be nonzero", who);
    const int64_t planes64 = static_cast<int64_t>(N) * C;
    const int64_t hw64 = static_cast<int64_t>(H) * W;
    if (planes64 > 0x7fffffffLL || hw64 > (1 << 24) || planes64 * hw64 > 0x7fffffffLL)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: N*C=%lld or H*W=%lld too large", who, (long long)planes64, (long long)hw64);
    if (N > 65535) return fail(SNNF_ERR_UNSUPPORTED, "%s: N=%d exceeds 65535", who, N);
    if (static_cast<size_t>(C) * sizeof(float) > 64 * 1024)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: C=%d exceeds LDS capacity", who, C);
    StepPtrs ptrs = {};
    for (int t = 0; t < T; ++t) {
        if (xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: xs[%d] is null", who, t);
        ptrs.p[t] = xs[t];
    }
    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    hipStream_t hs = as_stream(stream);
    const int planes = static_cast<int>(planes64);
    const int HW = static_cast<int>(hw64);

    // Small tails: one launch (a workgroup per sample and class range), when every operand allows 16-byte accesses.
    {
        bool aligned = aligned_to(v_out, 16) && (v_init == nullptr || aligned_to(v_init, 16)) && aligned_to(fc_weight, 16);
        for (int t = 0; t < T; ++t) aligned = aligned && aligned_to(xs[t], 16);
        const int class_blocks = aligned ? one_launch_class_blocks(T, N, C, HW, K) : 0;
        if (class_blocks > 0) {
            const dim3 grid(class_blocks, N);
            const int per_block = (K + class_blocks - 1) / class_blocks;
            const float inv_hw = 1.0f / static_cast<float>(HW);
            const float steps = static_cast<float>(T);
#define SNNF_TAIL_ONE(XT, VT)                                                                                               \
    lif_pool_linear_one_kernel<XT, VT><<<grid, kThreads, 0, hs>>>(ptrs, T, C, HW, K, per_block, static_cast<const VT*>(v_init), \
                                                                  static_cast<VT*>(v_out), static_cast<const XT*>(fc_weight),   \
                                                                  static_cast<const XT*>(fc_bias), static_cast<XT*>(out_sum), lif, inv_hw, steps)
            if (x_dtype == SNNF_F32) SNNF_TAIL_ONE(float, float);
            else if (x_dtype == SNNF_BF16) {
                if (v_dtype == SNNF_F32) SNNF_TAIL_ONE(bf16_t, float);
                else SNNF_TAIL_ONE(bf16_t, bf16_t);
            } else {
                if (v_dtype == SNNF_F32) SNNF_TAIL_ONE(f16_t, float);
                else SNNF_TAIL_ONE(f16_t, f16_t);
            }
#undef SNNF_TAIL_ONE
            return check_launch(who);
        }
    }

    int rc;
    if (x_dtype == SNNF_F32) rc = run<float, float>(ptrs, T, planes, HW, v_init, v_out, counts, lif, hs);
    else if (x_dtype == SNNF_BF16)
        rc = v_dtype == SNNF_F32 ? run<bf16_t, float>(ptrs, T, planes, HW, v_init, v_out, counts, lif, hs)
                                 : run<bf16_t, bf16_t>(ptrs, T, planes, HW, v_init, v_out, counts, lif, hs);
    else
        rc = v_dtype == SNNF_F32 ? run<f16_t, float>(ptrs, T, planes, HW, v_init, v_out, counts, lif, hs)
                                 : run<f16_t, f16_t>(ptrs, T, planes, HW, v_init, v_out, counts, lif, hs);
    if (rc != SNNF_OK) return rc;

    const int rows_per_block = (kThreads / 64) * kRowsPerWave;
    const dim3 grid((K + rows_per_block - 1) / rows_per_block, N);
    const size_t lds = static_cast<size_t>(C) * sizeof(float);
    const float inv_hw = 1.0f / static_cast<float>(HW);
    const float steps = static_cast<float>(T);
    const bool vec = C % kVec == 0 && aligned_to(fc_weight, 16);
    const bool matrix = vec && x_dtype != SNNF_F32 && C % 32 == 0 && N >= kMmMinSamples && K >= kMmMinClasses && static_cast<int64_t>(T) * HW <= kMmMaxCount;
    if (x_dtype == SNNF_F32) run_linear<float>(vec, false, grid, lds, hs, counts, C, K, fc_weight, fc_bias, out_sum, inv_hw, steps);
    else if (x_dtype == SNNF_BF16) run_linear<bf16_t>(vec, matrix, grid, lds, hs, counts, C, K, fc_weight, fc_bias, out_sum, inv_hw, steps);
    else run_linear<f16_t>(vec, matrix, grid, lds, hs, counts, C, K, fc_weight, fc_bias, out_sum, inv_hw, steps);
    return check_launch(who);
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_lif_pool_linear(const void* const* xs, int T, int N, int C, int H, int W, int x_dtype,
                                    const void* v_init, int v_dtype, const void* fc_weight, const void* fc_bias, int K,
                                    int w_dtype, void* out_sum, void* v_out, void* workspace, size_t workspace_bytes,
                                    float v_threshold, float v_reset, float tau, void* stream) {
    using namespace snnf;
    if (xs == nullptr || fc_weight == nullptr || out_sum == nullptr || v_out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_pool_linear: xs, fc_weight, out_sum and v_out must be non-null");
    if (T < 1 || N < 1 || C < 1 || H < 1 || W < 1 || K < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_pool_linear: T=%d N=%d C=%d H=%d W=%d K=%d", T, N, C, H, W, K);
    if (workspace == nullptr || workspace_bytes < snnf_lif_pool_linear_workspace_bytes(N, C) || !aligned_to(workspace, 16))
        return fail(SNNF_ERR_WORKSPACE, "snnf_lif_pool_linear: workspace of %zu bytes (16-byte aligned) required",
                    snnf_lif_pool_linear_workspace_bytes(N, C));
    return lif_pool_linear_impl("snnf_lif_pool_linear", xs, T, N, C, H, W, x_dtype, v_init, v_dtype, fc_weight, fc_bias, K, w_dtype,
                                out_sum, v_out, static_cast<int*>(workspace), v_threshold, v_reset, tau, stream);
}

extern "C" int snnf_spike_pool_linear(const void* const* spikes, int T, int N, int C, int H, int W, const void* fc_weight,
                                      const void* fc_bias, int K, int w_dtype, void* out, float out_scale, void* stream) {
    using namespace snnf;
    const char* who = "snnf_spike_pool_linear";
    if (spikes == nullptr || fc_weight == nullptr || out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: spikes, fc_weight and out must be non-null", who);
    if (T < 1 || N < 1 || C < 1 || H < 1 || W < 1 || K < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: T=%d N=%d C=%d H=%d W=%d K=%d", who, T, N, C, H, W, K);
    if (T > SNNF_MAX_T_PER_LAUNCH)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_temporal_length: T=%d exceeds %d", who, T, SNNF_MAX_T_PER_LAUNCH);
    if (w_dtype != SNNF_BF16 && w_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_dtype: bfloat16 or float16 classifier (the dtype of the result)", who);
    if (C % 8 != 0 || C > kOneMaxC || N > 65535)
        return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_shape: %d channels (whole groups of 8, at most %d) of %d samples (at most 65535)", who, C, kOneMaxC, N);
    if (!aligned_to(fc_weight, 16) || !aligned_to(out, 2) || (fc_bias != nullptr && !aligned_to(fc_bias, 2)))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: fc_weight must be 16-byte aligned, fc_bias and out element aligned", who);
    for (int t = 0; t < T; ++t)
        if (spikes[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "%s: spikes[%d] is null", who, t);
    // The timesteps of a bit-packed tensor lie at equal distances (one allocation): the kernel walks them by a stride.
    const int64_t step_stride = T > 1 ? static_cast<const unsigned char*>(spikes[1]) - static_cast<const unsigned char*>(spikes[0]) : 0;
    for (int t = 1; t < T; ++t)
        if (static_cast<const unsigned char*>(spikes[t]) - static_cast<const unsigned char*>(spikes[t - 1]) != step_stride)
            return fail(SNNF_ERR_UNSUPPORTED, "%s: unsupported_layout: the timesteps must lie at equal distances in memory", who);
    const unsigned char* base = static_cast<const unsigned char*>(spikes[0]);
    const int HW = H * W;
    const int C8 = C / 8;
    const int parts = std::max(1, std::min(HW, kThreads / std::max(1, C8)));   // threads that share a channel group's pixels
    const int rows_per_pass = (kThreads / 64) * kRowsPerWave;
    const int class_blocks = std::max(1, std::min((K + rows_per_pass - 1) / rows_per_pass, 512 / std::max(1, N)));
    const int per_block = (K + class_blocks - 1) / class_blocks;
    const dim3 grid(class_blocks, N);
    const float inv_hw = 1.0f / static_cast<float>(HW);
    hipStream_t hs = as_stream(stream);
    const int64_t sample_bytes = static_cast<int64_t>(C8) * HW;
    const bool staged = sample_bytes % 16 == 0 && T * sample_bytes <= kSpikeStageBytes && aligned_to(base, 16) && step_stride % 16 == 0;
#define SNNF_SPIKE_TAIL(XT, STAGED)                                                                                                         \
    spike_pool_linear_kernel<XT, STAGED><<<grid, kThreads, 0, hs>>>(base, step_stride, T, C8, HW, parts, K, per_block, static_cast<const XT*>(fc_weight), \
                                                                    static_cast<const XT*>(fc_bias), static_cast<XT*>(out), inv_hw,          \
                                                                    static_cast<float>(T), out_scale)
    if (w_dtype == SNNF_BF16) {
        if (staged) SNNF_SPIKE_TAIL(bf16_t, true);
        else SNNF_SPIKE_TAIL(bf16_t, false);
    } else {
        if (staged) SNNF_SPIKE_TAIL(f16_t, true);
        else SNNF_SPIKE_TAIL(f16_t, false);
    }
#undef SNNF_SPIKE_TAIL
    return check_launch(who);
}

// ---------------------------------------------------------------------------------------------------------------
// The same operator for callers that cannot allocate: the spike counts live in a static device array of the library.
// ---------------------------------------------------------------------------------------------------------------
namespace snnf {
namespace {

constexpr int kStaticCounts = SNNF_LIF_POOL_LINEAR_STATIC_MAX_PLANES;   // N * C of one call, at most
constexpr int kMaxDevices = 64;

// One copy per GPU the library runs on, held until the process ends. In host code this name is only a handle for
// hipGetSymbolAddress: the device address it yields is what kernels and memory calls get.
static __device__ __align__(256) int scratch[kStaticCounts];

// Device address of `scratch` on the current device (looked up once per device), or nullptr after reporting why not.
int* static_counts() {
    static std::mutex mu;
    static int* address[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        fail(SNNF_ERR_LAUNCH, "snnf_lif_pool_linear_static: cannot identify the current device");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (address[dev] == nullptr) {
        void* p = nullptr;
        const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || p == nullptr) {
            fail(SNNF_ERR_LAUNCH, "snnf_lif_pool_linear_static: hipGetSymbolAddress failed: %s", hipGetErrorString(err));
            return nullptr;
        }
        address[dev] = static_cast<int*>(p);
    }
    return address[dev];
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_lif_pool_linear_static(const void* const* xs, int T, int N, int C, int H, int W, int x_dtype,
                                           const void* v_init, int v_dtype, const void* fc_weight, const void* fc_bias,
                                           int K, int w_dtype, void* out_sum, void* v_out,
                                           float v_threshold, float v_reset, float tau, void* stream) {
    using namespace snnf;
    if (xs == nullptr || fc_weight == nullptr || out_sum == nullptr || v_out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_pool_linear_static: xs, fc_weight, out_sum and v_out must be non-null");
    if (T < 1 || N < 1 || C < 1 || H < 1 || W < 1 || K < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_pool_linear_static: T=%d N=%d C=%d H=%d W=%d K=%d", T, N, C, H, W, K);
    if (static_cast<int64_t>(N) * C > kStaticCounts)
        return fail(SNNF_ERR_WORKSPACE, "snnf_lif_pool_linear_static: N*C=%lld exceeds the static scratch of %d planes; "
                    "use snnf_lif_pool_linear with a workspace", static_cast<long long>(N) * C, kStaticCounts);
    int* counts = static_counts();
    if (counts == nullptr) return SNNF_ERR_LAUNCH;
    // Every plane count the second launch reads is written by the first, so nothing of an earlier call needs clearing.
    return lif_pool_linear_impl("snnf_lif_pool_linear_static", xs, T, N, C, H, W, x_dtype, v_init, v_dtype, fc_weight, fc_bias, K,
                                w_dtype, out_sum, v_out, counts, v_threshold, v_reset, tau, stream);
}
