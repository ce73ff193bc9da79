#!/usr/bin/env python3
"""Benchmark of the block-sparse linear hot path on one MI355X.

One step = forward Y = X.W^T, input gradient dX = dY.W and weight gradient dW = dY^T.X on the
sparse support, for BlockSparseLinear(4096 -> 4096, density 0.25), 16384 tokens, bf16 operands
with fp32 accumulation.  Inputs are synthetic (seeded) and resident in HBM before timing starts.

Prints ONE JSON line: effective TFLOP/s (2*M*nnz*1024 per GEMM, 3 GEMMs per step) with
  roofline       the slowest of the three kernels against the MI355X dense MFMA peak of the dtype,
  dense_hipblaslt  the same three GEMMs dense through torch.matmul (hipBLASLt) at the same shape,
  cpu_baseline   the CPU dense-equivalent path (oracle) timed on the host cores, full size,
  other_configs  the other benchmark configurations (1024->256 forward, the two RoBERTa feed-forward
                 shapes in fp32, the 4096 x 4096 layer in fp32 and at density 0.5 in both dtypes, the RoBERTa-base
                 training step), each with its own dense comparison.

Timing: after a settling phase and `--warmup` untimed steps, exactly `--steps` steps are timed between two
synchronisations; an event is recorded after every kernel of every timed step.  `ms_per_step` and `value`
are the median over the timed steps (the mean over the same region is `ms_per_step_mean`).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}  # MI355X dense matrix peaks
HBM_TBPS = 8.0

# HBM bytes per launch (fetch + write) of each kernel come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script (counters cannot be read from inside the process).  They are kept in profiles/traffic.json
# together with a hash of the kernel sources they were measured on; a figure measured on other sources is
# not reported (null).
BASELINE_WORKLOAD = "c4_4096x4096_d0.25_bf16"
BASELINE_METRIC = "effective TFLOP/s fwd+bwd at 4096² d=0.25; % of MFMA peak; vs dense GEMM"   # as in BASELINE.json
OTHER_LAYER_WORKLOADS = ("c1_1024x256_d0.1_fp32", "c2_768x3072_d0.5_fp32", "c3_3072x768_d0.25_zipf_fp32",
                         "c4_4096x4096_d0.25_fp32",   # the headline shape in the reference's own dtype
                         # and at the upper end of the density range the speed-up over dense is asked for
                         "c4_4096x4096_d0.5_bf16", "c4_4096x4096_d0.5_fp32")
ROBERTA_WORKLOAD = "c5_roberta_base_mlm_fp32"


def kernel_source_hash():
    """sha256 over the kernel sources, in name order."""
    import glob
    import hashlib

    h = hashlib.sha256()
    src = os.path.join(ROOT, "pytorch_block_sparse_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(src, "*.h")) + glob.glob(os.path.join(src, "*.hip"))):
        h.update(os.path.basename(path).encode())
        h.update(open(path, "rb").read())
    return h.hexdigest()


def measured_traffic(workload, tokens, kernel):
    """Bytes per launch from profiles/traffic.json, or None if absent or measured on other kernel sources."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    rec = json.load(open(path))
    if rec.get("kernel_source_sha256") != kernel_source_hash():
        return None
    return rec.get("bytes_per_launch", {}).get(f"{workload}@{tokens}", {}).get(kernel)


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--workload", default=BASELINE_WORKLOAD)
    p.add_argument("--tokens", type=int, default=None, help="override the workload's token count")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-dense", action="store_true", help="skip the dense hipBLASLt leg")
    p.add_argument("--no-others", action="store_true", help="skip the other_configs leg (C1, C2, C3, RoBERTa step)")
    p.add_argument("--cpu-sample-tokens", type=int, default=None, help="tokens of the CPU baseline leg (default: all)")
    p.add_argument("--copy-calibration", action="store_true",
                   help="also run a plain 256 MiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    return p.parse_args()


def median(v):
    v = sorted(v)
    n = len(v)
    return v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])


def settle(fn, seconds=0.3):
    """Untimed: run fn until `seconds` have passed, so that clocks and caches are past their start-up transient."""
    import torch

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(5):
            fn()
        torch.cuda.synchronize()


def time_steps(kernels, steps, warmup):
    """kernels: ordered {name: callable}.  Returns (median ms per step, mean ms per step, median ms per kernel)."""
    import torch

    def step():
        for f in kernels.values():
            f()

    settle(step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    names = list(kernels)
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(names) + 1)] for _ in range(steps)]
    for i in range(steps):
        marks[i][0].record()
        for j, kname in enumerate(names):
            kernels[kname]()
            marks[i][j + 1].record()
    torch.cuda.synchronize()
    per_step = [marks[i][0].elapsed_time(marks[i][-1]) for i in range(steps)]
    mean_ms = marks[0][0].elapsed_time(marks[-1][-1]) / steps
    per_kernel = {
        kname: median([marks[i][j].elapsed_time(marks[i][j + 1]) for i in range(steps)]) for j, kname in enumerate(names)
    }
    return median(per_step), mean_ms, per_kernel


def forward_latency(call, n_graph=20):
    """Latency figures of a small forward product, in microseconds per call: `host_issue` = wall time of back-to-back
    calls without synchronisation (what the Python + ctypes path costs; the GPU keeps up), `graph_replay` = the call
    captured n_graph times into one HIP graph and replayed (kernel time plus the gap between two launches, no host
    path), next to the event figure of time_steps (launch latency + kernel)."""
    import torch

    for _ in range(20):
        call()
    torch.cuda.synchronize()
    n = 1000
    t0 = time.perf_counter()
    for _ in range(n):
        call()
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(n_graph):
            keep = call()
    for _ in range(5):
        graph.replay()
    torch.cuda.synchronize()
    per = []
    for _ in range(50):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        per.append(e0.elapsed_time(e1) / n_graph * 1e3)
    del keep
    return {"host_issue": (t1 - t0) / n * 1e6, "graph_replay": median(per)}


def cpu_baseline(w, tokens):
    """The reference's CPU dense-equivalent path (to_dense + matmul, fp32): 3 warm-up + 5 timed runs, median."""
    import torch

    from oracle import block_sparse_oracle as O
    from pytorch_block_sparse_amd import workloads

    blocks, data, x, dy = workloads.make_inputs(w, tokens=tokens)
    X, Y = w.grid
    mask = O.mask_from_blocks(X, Y, blocks)
    idx = O.build_indices(mask)
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    shape = (w.out_features, w.in_features)
    w_dense = torch.from_numpy(O.to_dense(data.float().numpy(), coo, shape))
    mask_dense = torch.from_numpy(O.block_mask_dense(coo, shape)).float()
    xf, dyf = x.float(), dy.float()
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    for _ in range(3):
        O.linear_fwd_bwd_torch_fp32(xf, dyf, w_dense, mask_dense)
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        O.linear_fwd_bwd_torch_fp32(xf, dyf, w_dense, mask_dense)
        times.append(time.perf_counter() - t0)
    med = median(times)
    eff = 3 * 2.0 * tokens * w.nnz * 1024 / med / 1e12
    what = "all" if tokens == w.tokens else f"first {tokens} of"
    return {
        "value": eff,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{what} {w.tokens} tokens, same layer; torch CPU fp32 dense-equivalent fwd+dX+dW, "
        f"3 warm-up + 5 timed runs, median {med * 1e3:.1f} ms",
    }


def measure_layer(w, tokens, steps, warmup, dense=True):
    """Times the GEMMs of one BlockSparseLinear workload; returns the figures the JSON line is built from."""
    import torch

    from pytorch_block_sparse_amd import BlockSparseMatrix, workloads

    dev = torch.device("cuda:0")
    blocks, data, x, dy = workloads.make_inputs(w, tokens=tokens)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(dev)
    xd, dyd = x.to(dev), dy.to(dev)
    torch.cuda.synchronize()
    kernels = {"fwd": lambda: m.reverse_matmul(xd, True)}
    if w.passes != "fwd":
        kernels["dx"] = lambda: m.reverse_matmul(dyd, False)
        kernels["dw"] = lambda: m.matmul_with_output_sparse_support(dyd, xd)
    ms_step, ms_mean, per_kernel = time_steps(kernels, steps, warmup)
    dname = "bf16" if w.dtype == torch.bfloat16 else "f32"
    flops_gemm = 2.0 * tokens * w.nnz * 1024
    res = {
        "dtype": dname,
        "tokens": tokens,
        "n_gemms": len(kernels),
        "flops_gemm": flops_gemm,
        "ms_per_step": ms_step,
        "ms_per_step_mean": ms_mean,
        "kernel_ms": per_kernel,
        "value": len(kernels) * flops_gemm / (ms_step * 1e-3) / 1e12,
    }
    if w.passes == "fwd":
        res["latency_us"] = forward_latency(kernels["fwd"])
    if dense:
        wd = m.to_dense()
        dk = {"fwd": lambda: xd @ wd.t()}
        if w.passes != "fwd":
            dk["dx"] = lambda: dyd @ wd
            dk["dw"] = lambda: dyd.t() @ xd
        ms_dense, _, _ = time_steps(dk, steps, warmup)
        res["dense"] = {
            "ms_per_step": ms_dense,
            "dense_tflops": len(dk) * 2.0 * tokens * w.in_features * w.out_features / (ms_dense * 1e-3) / 1e12,
            "speedup_sparse_vs_dense": ms_dense / ms_step,
        }
    return res


def measure_roberta(steps, warmup):
    """One MLM training step (forward + backward + AdamW, fp32) of a 12-layer RoBERTa-base-shaped encoder
    with random weights, batch 32 x 512 random token ids, once with dense linear layers and once with
    attention.output.dense, intermediate.dense and output.dense of every layer patched to block-sparse
    layers of density 0.5 (the reference's tests/test_integration.py:66-113 procedure at full size)."""
    import torch
    from transformers import RobertaConfig, RobertaForMaskedLM

    from pytorch_block_sparse_amd import BlockSparseLinear, BlockSparseModelPatcher

    dev = torch.device("cuda:0")
    batch, seq = 32, 512
    cfg = RobertaConfig(vocab_size=50265, hidden_size=768, num_hidden_layers=12, num_attention_heads=12,
                        intermediate_size=3072, max_position_embeddings=seq + 2,
                        hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size, (batch, seq), generator=g)
    labels = ids.clone()
    labels[torch.rand((batch, seq), generator=g) >= 0.15] = -100   # 15 % of the positions are predicted
    ids, labels = ids.to(dev), labels.to(dev)

    def build(sparse):
        torch.manual_seed(1)
        model = RobertaForMaskedLM(cfg)
        n_dense = sum(p.numel() for p in model.parameters())
        model = model.to(dev)
        n_layers = 0
        if sparse:
            import contextlib
            import io

            mp = BlockSparseModelPatcher()
            for pat in (r"roberta\.encoder\.layer\.[0-9]+\.attention\.output\.dense",
                        r"roberta\.encoder\.layer\.[0-9]+\.intermediate\.dense",
                        r"roberta\.encoder\.layer\.[0-9]+\.output\.dense"):
                mp.add_pattern(pat, {"density": 0.5})
            with contextlib.redirect_stdout(io.StringIO()):   # the patcher prints one line per layer
                mp.patch_model(model)
            n_layers = sum(isinstance(m, BlockSparseLinear) for m in model.modules())
        return model, n_dense, sum(p.numel() for p in model.parameters()), n_layers

    def time_model(model):
        opt = torch.optim.AdamW(model.parameters(), lr=1e-4)

        def one():
            loss = model(input_ids=ids, labels=labels).loss
            loss.backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
            return loss

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        marks[0].record()
        for i in range(steps):
            loss = one()
            marks[i + 1].record()
        torch.cuda.synchronize()
        return median([marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]), float(loss.detach())

    model, n_dense, _, _ = build(False)
    ms_dense, loss_dense = time_model(model)
    del model
    torch.cuda.empty_cache()
    model, _, n_sparse, n_layers = build(True)
    ms_sparse, loss_sparse = time_model(model)
    del model
    torch.cuda.empty_cache()
    return {
        "batch": batch, "seq_len": seq, "patched_layers": n_layers, "steps": steps, "warmup": warmup,
        "dense_model": {"ms_per_step": ms_dense, "parameters": n_dense, "loss": loss_dense},
        "sparse_model": {"ms_per_step": ms_sparse, "parameters": n_sparse, "loss": loss_sparse},
        "tokens_per_s": batch * seq / (ms_sparse * 1e-3),
        "speedup_sparse_vs_dense": ms_dense / ms_sparse,
    }


def roberta_line(args):
    r = measure_roberta(args.steps, args.warmup)
    print(json.dumps({
        "metric": "MLM training step of a RoBERTa-base-shaped encoder, 36 linear layers block-sparse at density 0.5",
        "value": r["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": r["sparse_model"]["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": ROBERTA_WORKLOAD, "layers": 12, "hidden": 768, "ffn": 3072, "vocab": 50265,
                   "batch": r["batch"], "seq_len": r["seq_len"], "density": 0.5, "patched_layers": r["patched_layers"]},
        "dense_model": r["dense_model"],
        "sparse_model": r["sparse_model"],
        "speedup_sparse_vs_dense": r["speedup_sparse_vs_dense"],
    }))


def kernel_label(w, tokens, which):
    """The kernel(s) the library runs for this GEMM, as the library itself reports them."""
    from pytorch_block_sparse_amd import native

    if which == "dw":
        return native.matmul_back_kernel_name(tokens, w.out_features, w.in_features, w.nnz, w.dtype)
    n, k, transpose = (w.out_features, w.in_features, True) if which == "fwd" else (w.in_features, w.out_features, False)
    return native.matmul_kernel_name(tokens, n, k, w.nnz, transpose, w.dtype) + ("<forward>" if transpose else "<input gradient>")


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    import torch

    from pytorch_block_sparse_amd import native, workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    native.load()  # fail loudly if the HIP library is not built
    if args.workload == ROBERTA_WORKLOAD:
        roberta_line(args)
        return
    w = workloads.WORKLOADS[args.workload]
    tokens = args.tokens or w.tokens
    r = measure_layer(w, tokens, args.steps, args.warmup, dense=not args.no_dense)
    dname, per_kernel, flops_gemm = r["dtype"], r["kernel_ms"], r["flops_gemm"]
    dom = max(per_kernel, key=per_kernel.get)
    achieved = flops_gemm / (per_kernel[dom] * 1e-3) / 1e12
    # which roofline bounds the kernel: time at the matrix peak against time at the HBM peak for the algorithmic bytes
    e = 2 if dname == "bf16" else 4
    alg_bytes = e * (tokens * w.in_features + tokens * w.out_features + w.nnz * 1024)
    t_mfma = flops_gemm / (PEAK_TFLOPS[dname] * 1e12)
    t_hbm = alg_bytes / (HBM_TBPS * 1e12)

    out = {
        "metric": BASELINE_METRIC if w.name == BASELINE_WORKLOAD and tokens == w.tokens
        else f"effective TFLOP/s of the block-sparse GEMMs ({w.passes}) of {w.name} at {tokens} tokens",
        "value": r["value"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": r["ms_per_step"],
        "ms_per_step_mean": r["ms_per_step_mean"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dname,
        "data": "synthetic",
        "config": {
            "workload": w.name,
            "in_features": w.in_features,
            "out_features": w.out_features,
            "density": w.density,
            "nnz_blocks": w.nnz,
            "tokens": tokens,
            "pattern": w.pattern,
            "passes": w.passes,
        },
        "pct_of_mfma_peak": 100.0 * r["value"] / PEAK_TFLOPS[dname],
        "kernel_ms": per_kernel,
        "kernel_eff_tflops": {k: flops_gemm / (v * 1e-3) / 1e12 for k, v in per_kernel.items()},
        "roofline": {
            "bound": "mfma" if t_mfma >= t_hbm else "hbm",
            "kernel": kernel_label(w, tokens, dom),
            "achieved": achieved,
            "peak": PEAK_TFLOPS[dname],
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_TFLOPS[dname],
            "traffic": measured_traffic(w.name, tokens, dom),
            "traffic_unit": "bytes per launch",
            "flops_per_launch": flops_gemm,
            "algorithmic_bytes_per_launch": alg_bytes,
        },
    }
    if "dense" in r:
        out["dense_hipblaslt"] = r["dense"]
    if "latency_us" in r:
        out["latency_us"] = r["latency_us"]

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration_bytes"] = 1 << 28

    if not args.no_others and w.name == BASELINE_WORKLOAD and tokens == w.tokens:
        others = {}
        for name in OTHER_LAYER_WORKLOADS:
            ow = workloads.WORKLOADS[name]
            o = measure_layer(ow, ow.tokens, 30, 10, dense=not args.no_dense)
            peak = PEAK_TFLOPS[o["dtype"]]
            slow = max(o["kernel_ms"], key=o["kernel_ms"].get)
            others[name] = {
                "ms_per_step": o["ms_per_step"],
                "value": o["value"],
                "unit": "TFLOP/s",
                "frac": o["flops_gemm"] / (o["kernel_ms"][slow] * 1e-3) / 1e12 / peak,   # slowest kernel against the matrix peak of its dtype
                "pct_of_mfma_peak": 100.0 * o["value"] / peak,
                "kernel_ms": o["kernel_ms"],
                **({"latency_us": o["latency_us"]} if "latency_us" in o else {}),
                "kernels": {k: kernel_label(ow, ow.tokens, k) for k in o["kernel_ms"]},
                "dense_ms_per_step": o["dense"]["ms_per_step"] if "dense" in o else None,
                "vs_dense": o["dense"]["speedup_sparse_vs_dense"] if "dense" in o else None,
            }
        try:
            rb = measure_roberta(5, 2)
            others[ROBERTA_WORKLOAD] = {
                "ms_per_step": rb["sparse_model"]["ms_per_step"],
                "value": rb["tokens_per_s"],
                "unit": "tokens/s",
                "dense_ms_per_step": rb["dense_model"]["ms_per_step"],
                "vs_dense": rb["speedup_sparse_vs_dense"],
                "patched_layers": rb["patched_layers"],
            }
        except ImportError as exc:   # transformers missing: the layer workloads above still stand
            others[ROBERTA_WORKLOAD] = {"skipped": str(exc)}
        out["other_configs"] = others

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_sample_tokens or tokens)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
