/*
 * Brute-force C restatement of the fused temporal SNN operators. TEST INFRASTRUCTURE ONLY: it pins
 * oracle/snn_oracle.py (and through it the HIP kernels) with textbook loops that share no code with PyTorch.
 * Only tests/, __graft_entry__ and bench.py's cpu_baseline leg may load the library built from this file.
 *
 * Follows pengjh0111/triton-snn-fusion runtime/snn_custom_ops.py:
 *   oracle_lif_scan          :384-409 scanned over T as in :521-536
 *   oracle_conv2d            the F.conv2d call of :426/:450/:514 (NCHW, OIHW, groups, dilation 1), float64 accumulate
 *   oracle_linear            the F.linear call of :577/:608, float64 accumulate
 *   oracle_avgpool_linear    :555-557 for one step: mean over HxW, then Linear
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off, so fp32 LIF arithmetic is not fused into FMAs).
 */
#include <stddef.h>
#include <stdint.h>

void oracle_lif_scan(const float* x_seq, int T, long numel, const float* v_init, float v_threshold, float v_reset,
                     float tau, float* spikes, float* v_out, float* h_out) {
    for (long i = 0; i < numel; ++i) {
        float v = v_init ? v_init[i] : 0.0f;
        for (int t = 0; t < T; ++t) {
            const float x = x_seq[(long)t * numel + i];
            float h;
            if (tau <= 1.0f) {
                h = v + x;
            } else {
                const float d = x - v;
                const float q = d / tau;
                h = v + q;
            }
            const int fired = h >= v_threshold;
            if (v_reset < 0.0f) {
                const float drop = (fired ? 1.0f : 0.0f) * v_threshold;
                v = h - drop;
            } else {
                v = fired ? v_reset : h;
            }
            spikes[(long)t * numel + i] = fired ? 1.0f : 0.0f;
            if (h_out) h_out[(long)t * numel + i] = h;
        }
        v_out[i] = v;
    }
}

void oracle_conv2d(const float* x, int N, int Cin, int H, int W, const float* w, int Cout, int KH, int KW,
                   const float* bias, int stride_h, int stride_w, int pad_h, int pad_w, int groups, float* out) {
    const int Ho = (H + 2 * pad_h - (KH - 1) - 1) / stride_h + 1;
    const int Wo = (W + 2 * pad_w - (KW - 1) - 1) / stride_w + 1;
    const int cin_g = Cin / groups;
    const int cout_g = Cout / groups;
    for (int n = 0; n < N; ++n)
        for (int oc = 0; oc < Cout; ++oc) {
            const int g = oc / cout_g;
            for (int oh = 0; oh < Ho; ++oh)
                for (int ow = 0; ow < Wo; ++ow) {
                    double acc = bias ? (double)bias[oc] : 0.0;
                    for (int ci = 0; ci < cin_g; ++ci)
                        for (int kh = 0; kh < KH; ++kh) {
                            const int ih = oh * stride_h - pad_h + kh;
                            if (ih < 0 || ih >= H) continue;
                            for (int kw = 0; kw < KW; ++kw) {
                                const int iw = ow * stride_w - pad_w + kw;
                                if (iw < 0 || iw >= W) continue;
                                const double xv = x[(((long)n * Cin + g * cin_g + ci) * H + ih) * W + iw];
                                const double wv = w[(((long)oc * cin_g + ci) * KH + kh) * KW + kw];
                                acc += xv * wv;
                            }
                        }
                    out[(((long)n * Cout + oc) * Ho + oh) * Wo + ow] = (float)acc;
                }
        }
}

void oracle_linear(const float* x, int M, int Fin, const float* w, int Fout, const float* bias, float* out) {
    for (int m = 0; m < M; ++m)
        for (int o = 0; o < Fout; ++o) {
            double acc = bias ? (double)bias[o] : 0.0;
            for (int k = 0; k < Fin; ++k) acc += (double)x[(long)m * Fin + k] * (double)w[(long)o * Fin + k];
            out[(long)m * Fout + o] = (float)acc;
        }
}

void oracle_avgpool_linear(const float* s, int N, int C, int HW, const float* w, int K, const float* bias,
                           float* out) {
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) {
            double acc = bias ? (double)bias[k] : 0.0;
            for (int c = 0; c < C; ++c) {
                double sum = 0.0;
                for (int p = 0; p < HW; ++p) sum += (double)s[((long)n * C + c) * HW + p];
                acc += (sum / (double)HW) * (double)w[(long)k * C + c];
            }
            out[(long)n * K + k] = (float)acc;
        }
}
