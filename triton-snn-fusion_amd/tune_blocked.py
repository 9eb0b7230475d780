"""Measures the launch choices of the blocked convolution + LIF kernel for the layers of the network configurations and
writes runtime/tuned_blocked_plans.json (read by runtime/hip_blocked_backend.py; layers not in it run on the planner).

    python triton-snn-fusion_amd/tune_blocked.py [--networks resnet18 vgg11] [--margin 0.03] [--out PATH]

Needs an MI355X. Per layer: every patch width x channel groups per stage x K-sharing waves the kernel accepts is timed
(20 launches captured into one HIP graph, best of 5 replays); a choice enters the table only when it beats the planner's
own by more than `--margin`, so that timing noise does not churn the table. The role of this file is that of the
reference's autotune sweep (kernels/benchmark_conv_lif_temporal_general.py:524-558), run ahead of time.
"""
from __future__ import annotations

import argparse
import importlib
import json
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
sys.path.insert(0, str(PKG_DIR.parent))


def _time_us(fn, torch, launches: int = 20, replays: int = 5) -> float:
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(launches):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1000.0 / launches)
    del graph
    return best


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--networks", nargs="+", default=["resnet18", "vgg11"], choices=["resnet18", "vgg11"])
    ap.add_argument("--margin", type=float, default=0.03)
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    import torch
    pkg = importlib.import_module("triton_snn_fusion_amd")
    W = importlib.import_module("triton_snn_fusion_amd.workloads")
    B = importlib.import_module("triton_snn_fusion_amd.runtime.hip_blocked_backend")
    del pkg
    out_path = Path(args.out) if args.out else B.TUNED_PLANS_PATH
    B.load_tuned_plans(Path("/nonexistent"))          # start from the planner everywhere
    dev, dtype, T = torch.device("cuda:0"), torch.bfloat16, 4
    g = torch.Generator(device="cpu")
    g.manual_seed(0)
    entries = []
    for net in args.networks:
        layers, batch = (W.RESNET18_LAYERS, W.RESNET18_BATCH) if net == "resnet18" else (W.VGG11_LAYERS, W.VGG11_BATCH)
        for name, cin, cout, size, k, stride, pad, _residual, analog, _count in layers:
            if analog:
                x = B.from_dense(torch.randn(batch, cin, size, size, generator=g).to(dev, dtype), B.C8, shared=True)
                x.T = T
            else:
                x = B.from_dense((torch.rand(T, batch, cin, size, size, generator=g) < 0.15).to(dev, dtype), B.BITS)
            w = (torch.randn(cout, cin, k, k, generator=g) * (2.0 / (cin * k * k)) ** 0.5).to(dev, dtype)
            b = (torch.randn(cout, generator=g) * 0.1).to(dev, dtype)
            lif = (1.0, 0.0, 2.0) if not (k == 1 and stride == 2) else None      # the shortcut convolutions have no neuron
            fn = lambda: B.conv_lif_blocked(x, w, b, [stride, stride], [pad, pad], lif, out_layout=B.BITS if lif else B.C8)
            key = B._plan_key(T, batch, cin, size, size, cout, k, k, stride, stride, pad, pad, analog)
            B.register_tuned_plan(key, 0, 0, 0)
            _time_us(fn, torch)                           # warm-up: clocks and caches settle before anything is compared
            base = _time_us(fn, torch)
            base_plan = B.last_conv_plan()
            if base_plan.get("kernel") == "plane_matrix":
                B.register_tuned_plan(key, 0, 0, 0)
                print(f"{net} {name}: {base:.2f} us as a matrix product per frame on the Linear + LIF kernel, nothing to choose", flush=True)
                continue
            wo = (size + 2 * pad - k) // stride + 1
            seen = {(base_plan.get("tile"), base_plan.get("stage_chunks"), base_plan.get("waves"))}
            best = (base, 0, 0, 0, base_plan)
            for pc in sorted({c for c in (1, 2, 4, 7, 8, 14, 16, 28, 32) if c <= wo}):
                for groups in (0, 2, 4, 8):
                    for waves in (0, 1, 2, 4, 8):
                        B.register_tuned_plan(key, pc, groups, waves)
                        try:
                            fn()
                        except RuntimeError:
                            continue
                        plan = B.last_conv_plan()
                        applied = int(plan.get("tuned", 0))
                        shape = (plan.get("tile"), plan.get("stage_chunks"), plan.get("waves"))
                        if not (applied & 1) or (waves and not (applied & 2)) or shape in seen:
                            continue                      # the kernel cannot run this choice on the shape, or it is a repeat
                        seen.add(shape)
                        us = _time_us(fn, torch)
                        if us < best[0]:
                            best = (us, pc, int(plan.get("stage_chunks", groups)) if groups else 0, waves, plan)
            # The winner against the planner once more, in turns (launch times drift by a few percent over a sweep).
            if best[1]:
                again_base, again_best = [], []
                for _ in range(3):
                    B.register_tuned_plan(key, 0, 0, 0)
                    again_base.append(_time_us(fn, torch))
                    B.register_tuned_plan(key, best[1], best[2], best[3])
                    again_best.append(_time_us(fn, torch))
                base, best = min(again_base), (min(again_best),) + best[1:]
            B.register_tuned_plan(key, 0, 0, 0)
            gain = 1.0 - best[0] / base
            print(f"{net} {name}: planner {base:.2f} us ({base_plan.get('tile')}, waves {base_plan.get('waves')}), best {best[0]:.2f} us "
                  f"(patch_cols={best[1]} stage_groups={best[2]} k_waves={best[3]}: {best[4].get('tile')}, waves {best[4].get('waves')}), "
                  f"gain {gain * 100:.1f} %", flush=True)
            if best[1] and gain > args.margin:
                entries.append({"network": net, "layer": name, "T": T, "N": batch, "Cin": cin, "H": size, "W": size, "Cout": cout,
                                "kernel": [k, k], "stride": [stride, stride], "padding": [pad, pad], "shared_frame": bool(analog),
                                "patch_cols": best[1], "stage_groups": best[2], "k_waves": best[3],
                                "us": round(best[0], 2), "planner_us": round(base, 2)})
    out_path.write_text(json.dumps({"device": torch.cuda.get_device_name(0), "dtype": "bf16", "margin": args.margin,
                                    "layers": entries}, indent=1) + "\n")
    print(f"wrote {len(entries)} entries to {out_path}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
