#!/usr/bin/env python3
"""Benchmark of the block-sparse linear hot path on one MI355X.

One step = forward Y = X.W^T, input gradient dX = dY.W and weight gradient dW = dY^T.X on the
sparse support, for BlockSparseLinear(4096 -> 4096, density 0.25), 16384 tokens, bf16 operands
with fp32 accumulation.  Inputs are synthetic (seeded) and resident in HBM before timing starts.

Prints ONE JSON line: effective TFLOP/s (2*M*nnz*1024 per GEMM, 3 GEMMs per step) with
  roofline      the slowest of the three kernels against the MI355X dense bf16 MFMA peak,
  dense         the same three GEMMs dense through torch.matmul (hipBLASLt) at the same shape,
  cpu_baseline  the CPU dense-equivalent path (oracle) timed on the host cores on a token sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}  # MI355X dense matrix peaks

# HBM bytes per launch (fetch + write) of each kernel, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script, scaled by what the same counters read for a plain 256 MiB device
# copy (fetch x2.0, write x1.0).  Counters cannot be read from inside the process, so the figures
# are recorded here per workload and token count; other workloads report null.
MIB = float(1 << 20)
MEASURED_TRAFFIC = {
    ("c4_4096x4096_d0.25_bf16", 16384): {
        "fwd": (413.5 + 128.0) * MIB,
        "dx": (385.5 + 128.0) * MIB,
        "dw": (385.8 + 64.0 + 64.0 + 8.0) * MIB,   # partial sums, then the reduction
    },
}
BASELINE_WORKLOAD = "c4_4096x4096_d0.25_bf16"
BASELINE_METRIC = "effective TFLOP/s fwd+bwd at 4096\u00b2 d=0.25; % of MFMA peak; vs dense GEMM"   # as in BASELINE.json


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--workload", default=BASELINE_WORKLOAD)
    p.add_argument("--tokens", type=int, default=None, help="override the workload's token count")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-dense", action="store_true", help="skip the dense hipBLASLt leg")
    p.add_argument("--cpu-sample-tokens", type=int, default=2048)
    p.add_argument("--copy-calibration", action="store_true",
                   help="also run a plain 256 MiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    return p.parse_args()


def time_gpu(fn, steps, warmup):
    """Average milliseconds per call of fn over `steps` calls, HIP events on the current stream."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def cpu_baseline(w, sample_tokens):
    """The reference's CPU dense-equivalent path (to_dense + matmul, fp32) on the first sample_tokens tokens."""
    import torch

    from oracle import block_sparse_oracle as O
    from pytorch_block_sparse_amd import workloads

    blocks, data, x, dy = workloads.make_inputs(w, tokens=sample_tokens)
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
    O.linear_fwd_bwd_torch_fp32(xf, dyf, w_dense, mask_dense)  # warm-up
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 and (len(times) < 2 or time.perf_counter() - t_all < 20.0):
        t0 = time.perf_counter()
        O.linear_fwd_bwd_torch_fp32(xf, dyf, w_dense, mask_dense)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    eff = 3 * 2.0 * sample_tokens * w.nnz * 1024 / med / 1e12
    return {
        "value": eff,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"first {sample_tokens} of {w.tokens} tokens, same layer; torch CPU fp32 dense-equivalent "
        f"fwd+dX+dW, median of {len(times)} runs ({med * 1e3:.1f} ms)",
    }


ROBERTA_WORKLOAD = "c5_roberta_base_mlm_fp32"


def run_roberta(args):
    """One MLM training step (forward + backward + AdamW, fp32) of a 12-layer RoBERTa-base-shaped encoder
    with random weights, batch 32 x 512 random token ids, once with dense linear layers and once with
    attention.output.dense, intermediate.dense and output.dense of every layer patched to block-sparse
    layers of density 0.5 (the reference's tests/test_integration.py:66-113 procedure at full size)."""
    import torch
    from transformers import RobertaConfig, RobertaForMaskedLM

    from pytorch_block_sparse_amd import BlockSparseLinear, BlockSparseModelPatcher, native

    native.load()
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
            mp = BlockSparseModelPatcher()
            for pat in (r"roberta\.encoder\.layer\.[0-9]+\.attention\.output\.dense",
                        r"roberta\.encoder\.layer\.[0-9]+\.intermediate\.dense",
                        r"roberta\.encoder\.layer\.[0-9]+\.output\.dense"):
                mp.add_pattern(pat, {"density": 0.5})
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

        for _ in range(args.warmup):
            one()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(args.steps):
            loss = one()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / args.steps, float(loss)

    model, n_dense, _, _ = build(False)
    ms_dense, loss_dense = time_model(model)
    del model
    torch.cuda.empty_cache()
    model, _, n_sparse, n_layers = build(True)
    ms_sparse, loss_sparse = time_model(model)
    tokens = batch * seq
    print(json.dumps({
        "metric": "MLM training step of a RoBERTa-base-shaped encoder, 36 linear layers block-sparse at density 0.5",
        "value": tokens / (ms_sparse * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_sparse,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": ROBERTA_WORKLOAD, "layers": 12, "hidden": 768, "ffn": 3072, "vocab": 50265,
                   "batch": batch, "seq_len": seq, "density": 0.5, "patched_layers": n_layers},
        "dense_model": {"ms_per_step": ms_dense, "parameters": n_dense, "loss": loss_dense},
        "sparse_model": {"ms_per_step": ms_sparse, "parameters": n_sparse, "loss": loss_sparse},
        "speedup_sparse_vs_dense": ms_dense / ms_sparse,
    }))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == ROBERTA_WORKLOAD:
        run_roberta(args)
        return
    import torch

    from pytorch_block_sparse_amd import BlockSparseMatrix, native, workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    native.load()  # fail loudly if the HIP library is not built
    dev = torch.device("cuda:0")
    w = workloads.WORKLOADS[args.workload]
    tokens = args.tokens or w.tokens
    blocks, data, x, dy = workloads.make_inputs(w, tokens=tokens)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(dev)
    xd, dyd = x.to(dev), dy.to(dev)
    torch.cuda.synchronize()

    def fwd():
        return m.reverse_matmul(xd, True)

    def dx():
        return m.reverse_matmul(dyd, False)

    def dw():
        return m.matmul_with_output_sparse_support(dyd, xd)

    if w.passes == "fwd":
        kernels = {"fwd": fwd}
    else:
        kernels = {"fwd": fwd, "dx": dx, "dw": dw}

    def step():
        for f in kernels.values():
            f()

    # The timed region is exactly `steps` steps.  Inside it an event is recorded after every kernel, so
    # that the per-kernel durations are those of the launches of the timed steps themselves (the same
    # launches a rocprofv3 kernel trace of this command averages), not of a kernel repeated on its own.
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    names = list(kernels)
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(names) + 1)] for _ in range(args.steps)]
    for i in range(args.steps):
        marks[i][0].record()
        for j, kname in enumerate(names):
            kernels[kname]()
            marks[i][j + 1].record()
    torch.cuda.synchronize()
    ms_step = marks[0][0].elapsed_time(marks[-1][-1]) / args.steps
    per_kernel = {
        kname: sum(marks[i][j].elapsed_time(marks[i][j + 1]) for i in range(args.steps)) / args.steps
        for j, kname in enumerate(names)
    }

    dname = "bf16" if w.dtype == torch.bfloat16 else "f32"
    flops_gemm = 2.0 * tokens * w.nnz * 1024
    n_gemms = len(kernels)
    value = n_gemms * flops_gemm / (ms_step * 1e-3) / 1e12
    dom = max(per_kernel, key=per_kernel.get)
    achieved = flops_gemm / (per_kernel[dom] * 1e-3) / 1e12
    sdd = "sdd_bf16_kernel" if dname == "bf16" else "sdd_kernel"

    def dds_name(n, k, trans):
        # the library picks the wide-tile kernel for bf16 when there are at least 256 tiles of 128 tokens x 512 columns
        wide = dname == "bf16" and k % 64 == 0 and ((tokens + 127) // 128) * ((n // 32 + 15) // 16) >= 256
        return ("dds16_kernel" if wide else "dds_kernel") + f"<TRANS={trans}>"

    kernel_names = {
        "fwd": dds_name(w.out_features, w.in_features, 0),
        "dx": dds_name(w.in_features, w.out_features, 1),
        "dw": sdd + " (+ sdd_reduce_kernel)",
    }
    traffic = MEASURED_TRAFFIC.get((w.name, tokens), {}).get(dom)

    out = {
        "metric": BASELINE_METRIC if w.name == BASELINE_WORKLOAD and tokens == w.tokens
        else f"effective TFLOP/s of the block-sparse GEMMs ({w.passes}) of {w.name} at {tokens} tokens",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
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
        "pct_of_mfma_peak": 100.0 * value / PEAK_TFLOPS[dname],
        "kernel_ms": per_kernel,
        "kernel_eff_tflops": {k: flops_gemm / (v * 1e-3) / 1e12 for k, v in per_kernel.items()},
        "roofline": {
            "bound": "mfma",
            "kernel": kernel_names[dom],
            "achieved": achieved,
            "peak": PEAK_TFLOPS[dname],
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_TFLOPS[dname],
            "traffic": traffic,
            "traffic_unit": "bytes per launch",
            "flops_per_launch": flops_gemm,
        },
    }

    if not args.no_dense:
        wd = m.to_dense()
        dense = {
            "fwd": lambda: xd @ wd.t(),
            "dx": lambda: dyd @ wd,
            "dw": lambda: dyd.t() @ xd,
        }
        if w.passes == "fwd":
            dense = {"fwd": dense["fwd"]}

        def dense_step():
            for f in dense.values():
                f()

        ms_dense = time_gpu(dense_step, args.steps, args.warmup)
        out["dense_hipblaslt"] = {
            "ms_per_step": ms_dense,
            "dense_tflops": n_gemms * 2.0 * tokens * w.in_features * w.out_features / (ms_dense * 1e-3) / 1e12,
            "speedup_sparse_vs_dense": ms_dense / ms_step,
        }
        del wd

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration_bytes"] = 1 << 28

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(w, min(args.cpu_sample_tokens, tokens))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
