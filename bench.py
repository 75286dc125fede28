#!/usr/bin/env python3
"""Benchmark of the kernel-fusion hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward + backward pass of the fused causal scale-mask-softmax
over one batch of synthetic attention scores: fp16 [8,16,2048,2048] ~ N(0,1)*8,
scale 0.125, upstream gradient ~ N(0,1). Inputs are resident in HBM before the
timed region. The JSON line printed at the end carries

  value         algorithmic bytes of a step / time of a step, in GB/s
  roofline      the causal forward kernel alone (its launches timed with events
                on the launch stream), as a fraction of the 8 TB/s HBM peak
  kernels       the same figure for every other kernel of the path at its
                benchmark shape
  cpu_baseline  the reference's unfused arithmetic on the host cores, timed on
                a bounded sample of the same workload

Algorithmic bytes count what the operation must move, not what the hardware
moved: forward = lower triangle read + full matrix written; backward = two
lower triangles read + full matrix written.
"""

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16, published
# Matrix products per visible (query, key) tile that the attention backward's
# passes issue when every pass computes the scores it needs, by head size
# (oslo_amd/csrc/attention_prefill_bwd.hip: the dQ pass 3, then dK and dV in
# one pass 4, or at 256 features, where both accumulators do not fit a lane's
# registers, 3 + 2 in two passes); the mathematics has 5, and so has the
# backward that hands P and dS from the dQ pass to the dK/dV pass through a
# tile store (what runs at 256 features).
BWD_PRODUCTS_ISSUED = {64: 7, 128: 7, 256: 8}

# HBM bytes per launch measured with `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` (KiB per dispatch, scaled by the reading of a 1 GiB copy
# kernel: 2.0 for FETCH_SIZE, 1.0 for WRITE_SIZE), as recorded in
# profiles/bench_kernels_hbm_traffic.md and, for the two kernels of the step,
# profiles/causal_softmax_fp16_8x16x2048x2048_hbm_traffic.md.
MEASURED_TRAFFIC = {
    "causal_fwd fp16 [8,16,2048,2048]": 1627471923,
    "causal_bwd fp16 [8,16,2048,2048]": 2181120048,
    "causal_fwd bf16 [8,16,2048,2048]": 1627459656,
    "causal_bwd bf16 [8,16,2048,2048] (in place)": 2181120137,
    "causal_dropout_fwd p=0.1 bf16 [8,16,2048,2048]": 1635900230,
    "causal_dropout_bwd p=0.1 bf16 [8,16,2048,2048] (in place)": 2214719499,
    "causal_fwd fp32 [8,16,2048,2048]": 3238067310,
    "causal_bwd fp32 [8,16,2048,2048] (in place)": 4328580363,
    "causal_fwd bf16 [1,16,8192,8192]": 3229695250,
    "masked_fwd bf16 [16,16,1024,1024] key mask": 1082271801,
    "masked_bwd bf16 [16,16,1024,1024]": 1610650634,
    "bias_gelu_fwd bf16 [16384,16384]": 1073877195,
    "bias_gelu_bwd+dbias bf16 [16384,16384]": 1677948106,
    "bias_dropout_add_fwd p=0.1 bf16 [16384,16384]": 1610758935,
    "bias_dropout_add_bwd+dbias p=0.1 bf16 [16384,16384]": 1141071052,
    "bias_gelu_fwd bf16 [16384,4096]": 268493535,
    "bias_gelu_bwd+dbias bf16 [16384,4096]": 419584379,
    "bias_dropout_add_fwd p=0.1 bf16 [16384,4096]": 402709849,
    "bias_dropout_add_bwd+dbias p=0.1 bf16 [16384,4096]": 285361737,
    "bias_dropout_add2_fwd (two residuals) p=0.1 bf16 [16384,4096]": 536945004,
    "bias_gelu_bwd without dbias bf16 [16384,4096]": 402744320,
    "bias_dropout_add_bwd without dbias p=0.1 bf16 [16384,4096]": 268517376,
    "rotary_qkv bf16 q,k,v [8,2048,16,256] rotary 64": 807985633,
    "causal_fwd bf16 [8,16,2048,2048] with padding mask": 1628022852,
    "causal_window_fwd window 256 bf16 [8,16,2048,2048]": 1230656581,
    "causal_window_bwd window 256 bf16 [8,16,2048,2048] (in place)": 1387504650,
    "causal_fwd bf16 [4,16,4096,4096]": 3238084608,
    "causal_bwd bf16 [4,16,4096,4096] (in place)": 4328603740,
    "linear_rows fc_in + bias + gelu bf16 1 x [16384,4096]": 134699022,
    "linear_rows fc_in + bias + gelu bf16 8 x [16384,4096]": 135284935,
    "linear_rows fc_out + bias bf16 1 x [4096,16384]": 134600960,
    "linear_rows fc_out + bias bf16 8 x [4096,16384]": 136611520,
    "linear_rows attention projection bf16 1 x [4096,4096]": 33740800,
    "linear_rows attention projection bf16 8 x [4096,4096]": 34370560,
    "attention_decode bf16 1 x 16 heads, 1024 of 1152 keys, head 256 (two launches)": 17573905,
    "attention_decode bf16 8 x 16 heads, 1024 of 1152 keys, head 256 (two launches)": 136477703,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gptj", action="store_true", help="skip the GPT-J-6B-shaped forward comparison")
    ap.add_argument("--only", default="",
                    help="run only the named kernel of the table, or one model-level pass "
                         "(gptj_fwd_fused, gptj_fwd_unfused, gptj_train_fused, gptj_train_unfused), for profiling")
    ap.add_argument("--zero-operands", action="store_true",
                    help="with --only attention_prefill or gemm: operands of zeros (clock and power readings)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; every softmax row and every "
                 "element is independent, so N GPUs would each run this same kernel on "
                 "1/N of the batch*heads with no exchange. Run with --gpus 1.")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm device visible")
    from oslo_amd import _lib

    lib = _lib.load()  # raises if the HIP library is not built; there is no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream()
    st = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.oslo_last_error().decode())

    def time_launches(fn, n, warm):
        """Average seconds per call of fn over n calls, events on the launch stream.
        Warm-up: `warm` calls and then until 30 ms have passed. After a change of
        workload the device's clocks take some milliseconds to settle (the same
        kernel on the same buffers was seen 15-25 % slower for its first few dozen
        launches after a set-up phase), and a kernel table is about the settled
        rate."""
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t_end = time.perf_counter() + 0.03
        while time.perf_counter() < t_end:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n

    # ---------------- workload: causal softmax fwd+bwd, fp16 [8,16,2048,2048]
    B, H, S = 8, 16, 2048
    F16, BF16 = 1, 2
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)
    x = (torch.randn((B, H, S, S), generator=gen, device=dev, dtype=torch.float32) * 8).to(torch.float16)
    gen.manual_seed(1)
    g = torch.randn((B * H, S, S), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
    y = torch.empty_like(x)
    dx = torch.empty_like(g)
    tri = B * H * S * (S + 1) // 2
    full = B * H * S * S
    bytes_fwd = 2 * (tri + full)
    bytes_bwd = 2 * (2 * tri + full)

    def fwd():
        check(lib.oslo_softmax_causal_fwd(P(y), P(x), None, 0.125, B, H, S, F16, st))

    def bwd():
        check(lib.oslo_softmax_causal_bwd(P(dx), P(g), P(y), 0.125, B * H, S, F16, st))

    def step():
        fwd()
        bwd()

    if args.only:
        run_only(args, lib, torch, dev, st, P, check, time_launches, fwd, bwd)
        return

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = (bytes_fwd + bytes_bwd) / (elapsed / args.steps) / 1e9

    t_fwd = time_launches(fwd, max(100, args.steps), 5)
    t_bwd = time_launches(bwd, max(100, args.steps), 5)

    def roof(name, nbytes, seconds, elements, buffer_sets=1):
        """elements: scores or activations the launch produces; buffer_sets:
        how many sets of tensors the timed launches took in turn."""
        gbps = nbytes / seconds / 1e9
        return {"kernel": name, "buffer_sets": buffer_sets, "elements_per_s": round(elements / seconds, 1), "bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "us": round(seconds * 1e6, 1),
                "algorithmic_bytes": nbytes, "traffic": MEASURED_TRAFFIC.get(name)}

    roofline = roof("causal_fwd fp16 [8,16,2048,2048]", bytes_fwd, t_fwd, full)
    kernels = [roof("causal_bwd fp16 [8,16,2048,2048]", bytes_bwd, t_bwd, full)]
    del x, y, g, dx
    kernels += other_kernels(lib, torch, dev, st, P, check, time_launches, roof, max(100, args.steps))

    out = {
        "metric": "fused causal scale-mask-softmax fwd+bwd HBM GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "causal scaled softmax fwd+bwd, fp16 scores [8,16,2048,2048], scale 0.125, "
                               "fp32 arithmetic",
                   "algorithmic_bytes_per_step": bytes_fwd + bytes_bwd},
        "roofline": roofline,
        "kernels": kernels,
    }
    def section(fn, *a):
        """A model-level section must not cost the line its kernel figures: what
        goes wrong in one is reported in its place."""
        try:
            return fn(*a)
        except Exception as e:  # noqa: BLE001
            torch.cuda.empty_cache()
            return {"error": f"{type(e).__name__}: {e}"[:300]}

    if not args.no_gptj:
        out["gptj_fwd"] = section(gptj_forward, torch, dev)
        out["gptj_train_step"] = section(gptj_train_step, torch, dev)
        # GPT-J's own setting, no attention dropout: the fused model trains through the one-kernel attention
        out["gptj_train_step_no_attention_dropout"] = section(gptj_train_step, torch, dev, 0.0)
        out["other_families_fwd"] = section(other_families_forward, torch, dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, section)
    # The figures a reader of the first kilobytes of the line needs, inside `config`: the second half
    # of the metric (GPT-J-shaped forward, tokens/s, unfused against fuse()), the training step, and
    # the fraction of its roofline of every kernel of the table.
    for key in ("gptj_fwd", "gptj_train_step"):
        sec = out.get(key)
        if isinstance(sec, dict):
            out["config"][key] = {k: sec[k] for k in ("unfused_tokens_per_s", "fused_tokens_per_s", "speedup",
                                                      "logits_vs_fp32", "error") if k in sec}
    out["config"]["kernel_fracs"] = {k["kernel"]: k["frac"] for k in kernels}
    print(json.dumps(out))


def other_kernels(lib, torch, dev, st, P, check, time_launches, roof, n):
    """Every other kernel of the path at its benchmark shape."""
    F16, BF16, F32 = 1, 2, 0
    res = []
    gen = torch.Generator(device=dev)

    def randn(shape, seed, std, dtype):
        gen.manual_seed(seed)
        return (torch.randn(shape, generator=gen, device=dev, dtype=torch.float32) * std).to(dtype)

    # causal, bf16 and fp32 variants of the workload
    B, H, S = 8, 16, 2048
    tri, full = B * H * S * (S + 1) // 2, B * H * S * S
    for name, dt, code in (("bf16", torch.bfloat16, BF16), ("fp32", torch.float32, F32)):
        x = randn((B, H, S, S), 0, 8.0, dt)
        y = torch.empty_like(x)
        es = x.element_size()
        t = time_launches(lambda: check(lib.oslo_softmax_causal_fwd(P(y), P(x), None, 0.125, B, H, S, code, st)), n, 3)
        res.append(roof(f"causal_fwd {name} [8,16,2048,2048]", es * (tri + full), t, full))
        g = randn((B * H, S, S), 1, 1.0, dt)
        t = time_launches(lambda: check(lib.oslo_softmax_causal_bwd(P(g), P(g), P(y), 0.125, B * H, S, code, st)), n, 3)
        res.append(roof(f"causal_bwd {name} [8,16,2048,2048] (in place)", es * (2 * tri + full), t, full))
        if name == "bf16":  # padded batches: additive key mask, lengths U{1024..2048}
            gen.manual_seed(2)
            lens = torch.randint(1024, S + 1, (B,), generator=gen, device=dev)
            pad = torch.where(torch.arange(S, device=dev)[None, :] < lens[:, None], 0.0, -10000.0).float().contiguous()
            t = time_launches(lambda: check(lib.oslo_softmax_causal_fwd(P(y), P(x), P(pad), 0.125, B, H, S, code, st)), n, 3)
            res.append(roof(f"causal_fwd {name} [8,16,2048,2048] with padding mask", es * (tri + full) + 4 * B * S, t, full))
        if name == "bf16":  # sliding-window rows (GPT-Neo local attention), window 256
            W = 256
            band = B * H * (W * (W + 1) // 2 + (S - W) * W)
            t = time_launches(lambda: check(lib.oslo_softmax_causal_window_fwd(
                P(y), P(x), None, 0.125, W, B, H, S, code, st)), n, 3)
            res.append(roof(f"causal_window_fwd window 256 {name} [8,16,2048,2048]", es * (band + full), t, full))
            t = time_launches(lambda: check(lib.oslo_softmax_causal_window_bwd(
                P(g), P(g), P(y), 0.125, W, B * H, S, code, st)), n, 3)
            res.append(roof(f"causal_window_bwd window 256 {name} [8,16,2048,2048] (in place)",
                            es * (2 * band + full), t, full))
            check(lib.oslo_softmax_causal_fwd(P(y), P(x), None, 0.125, B, H, S, code, st))
        if name == "bf16":  # training: attention dropout inside the softmax kernels
            stats = torch.empty((B * H * S, 2), dtype=torch.float32, device=dev)
            t = time_launches(lambda: check(lib.oslo_softmax_causal_dropout_fwd(
                P(y), P(stats), P(x), None, 0.125, 0.1, 1234, 0, B, H, S, code, st)), n, 3)
            res.append(roof(f"causal_dropout_fwd p=0.1 {name} [8,16,2048,2048]",
                            es * (tri + full) + 8 * B * H * S, t, full))
            t = time_launches(lambda: check(lib.oslo_softmax_causal_dropout_bwd(
                P(g), P(g), P(x), P(stats), None, 0.125, 0.1, 1234, 0, B, H, S, code, st)), n, 3)
            res.append(roof(f"causal_dropout_bwd p=0.1 {name} [8,16,2048,2048] (in place)",
                            es * (2 * tri + full) + 8 * B * H * S, t, full))
            del stats
        del x, y, g

    # long rows: bf16 [1,16,8192,8192]
    S8 = 8192
    x = randn((1, 16, S8, S8), 0, 1.0, torch.bfloat16)
    y = torch.empty_like(x)
    t = time_launches(lambda: check(lib.oslo_softmax_causal_fwd(P(y), P(x), None, 1 / 16, 1, 16, S8, BF16, st)), n, 3)
    res.append(roof("causal_fwd bf16 [1,16,8192,8192]", 2 * (16 * S8 * (S8 + 1) // 2 + x.numel()), t, x.numel()))
    del x, y

    # rows of 4096: bf16 [4,16,4096,4096], forward and backward (in place)
    S4 = 4096
    x = randn((4, 16, S4, S4), 0, 1.0, torch.bfloat16)
    y = torch.empty_like(x)
    tri4 = 64 * S4 * (S4 + 1) // 2
    t = time_launches(lambda: check(lib.oslo_softmax_causal_fwd(P(y), P(x), None, 1 / 16, 4, 16, S4, BF16, st)), n, 3)
    res.append(roof("causal_fwd bf16 [4,16,4096,4096]", 2 * (tri4 + x.numel()), t, x.numel()))
    g = randn((64, S4, S4), 1, 1.0, torch.bfloat16)
    t = time_launches(lambda: check(lib.oslo_softmax_causal_bwd(P(g), P(g), P(y), 1 / 16, 64, S4, BF16, st)), n, 3)
    res.append(roof("causal_bwd bf16 [4,16,4096,4096] (in place)", 2 * (2 * tri4 + x.numel()), t, x.numel()))
    del x, y, g

    # padded key mask: bf16 [16,16,1024,1024], lengths U{128..1024}
    B, H, S = 16, 16, 1024
    x = randn((B, H, S, S), 0, 8 ** 0.5, torch.bfloat16)
    y = torch.empty_like(x)
    gen.manual_seed(2)
    lens = torch.randint(128, 1025, (B,), generator=gen, device=dev)
    mask = (torch.arange(S, device=dev)[None, :] >= lens[:, None]).contiguous().view(torch.uint8)
    t = time_launches(lambda: check(lib.oslo_softmax_masked_fwd(P(y), P(x), P(mask), S, 0, 0, 0.125, B, H, S, S, BF16, st)), n, 3)
    res.append(roof("masked_fwd bf16 [16,16,1024,1024] key mask", 4 * x.numel() + mask.numel(), t, x.numel()))
    # the same with a [B,1,Sq,Sk] mask whose query rows past the sample's length are fully masked
    full_mask = (mask.view(B, 1, 1, S).bool() | (torch.arange(S, device=dev)[None, :] >= lens[:, None]).view(B, 1, S, 1))
    full_mask = full_mask.contiguous().view(torch.uint8)
    t = time_launches(lambda: check(lib.oslo_softmax_masked_fwd(P(y), P(x), P(full_mask), S * S, S, 0, 0.125, B, H, S, S, BF16, st)), n, 3)
    res.append(roof("masked_fwd bf16 [16,16,1024,1024] full [B,1,Sq,Sk] mask, fully masked tail rows",
                    4 * x.numel() + full_mask.numel(), t, x.numel()))
    del full_mask
    g = randn((B, H, S, S), 1, 1.0, torch.bfloat16)
    dxm = torch.empty_like(g)
    t = time_launches(lambda: check(lib.oslo_softmax_masked_bwd(P(dxm), P(g), P(y), 0.125, B * H * S, S, BF16, st)), n, 3)
    res.append(roof("masked_bwd bf16 [16,16,1024,1024]", 6 * x.numel(), t, x.numel()))
    del x, y, g, dxm

    def rotating(sets, call):
        """fn() that runs call(set) on the next of `sets` each time: a shape
        whose tensors fit the 256 MB last-level cache is timed on four sets of
        buffers in turn, so that no launch finds its input left there by the
        previous one."""
        turn = [0]

        def fn():
            call(sets[turn[0] % len(sets)])
            turn[0] += 1
        return fn

    # bias-GeLU and bias-dropout-residual, bf16
    for rows, cols in ((16384, 16384), (16384, 4096)):
        n_el = rows * cols
        n_sets = 1 if 6 * n_el >= (1 << 30) else 4
        sets = [(randn((rows, cols), 10 * i, 1.0, torch.bfloat16), randn((rows, cols), 10 * i + 1, 1.0, torch.bfloat16),
                 torch.empty((rows, cols), dtype=torch.bfloat16, device=dev),
                 randn((rows, cols), 10 * i + 2, 1.0, torch.bfloat16)) for i in range(n_sets)]
        bias = randn((cols,), 3, 0.02, torch.bfloat16)
        db = torch.empty_like(bias)
        ws = torch.empty(lib.oslo_colsum_workspace_bytes(rows, cols) // 4, dtype=torch.float32, device=dev)
        shape = f"bf16 [{rows},{cols}]"
        t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_gelu_fwd(
            P(b[2]), P(b[0]), P(bias), rows, cols, BF16, st))), n, 3)
        res.append(roof(f"bias_gelu_fwd {shape}", 4 * n_el, t, n_el, n_sets))
        t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_gelu_bwd(
            P(b[2]), P(db), P(ws), P(b[1]), P(b[0]), P(bias), rows, cols, BF16, st))), n, 3)
        res.append(roof(f"bias_gelu_bwd+dbias {shape}", 6 * n_el, t, n_el, n_sets))
        t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_dropout_add_fwd(
            P(b[2]), P(b[0]), P(bias), P(b[1]), 0.1, 1234, 0, rows, cols, BF16, st))), n, 3)
        res.append(roof(f"bias_dropout_add_fwd p=0.1 {shape}", 6 * n_el, t, n_el, n_sets))
        t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_dropout_add_bwd(
            P(b[2]), P(db), P(ws), P(b[1]), 0.1, 1234, 0, rows, cols, BF16, st))), n, 3)
        res.append(roof(f"bias_dropout_add_bwd+dbias p=0.1 {shape}", 4 * n_el, t, n_el, n_sets))
        if n_sets > 1:
            # GPT-J's three-term block sum in the same pass: dropout(x + bias) + residual + a second residual
            t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_dropout_add2_fwd(
                P(b[2]), P(b[0]), P(bias), P(b[1]), P(b[3]), 0.1, 1234, 0, rows, cols, BF16, st))), n, 3)
            res.append(roof(f"bias_dropout_add2_fwd (two residuals) p=0.1 {shape}", 8 * n_el, t, n_el, n_sets))
            # without the bias gradient (one launch, no partial rows): what the second launch and the
            # partial rows of the rows above cost at this size
            t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_gelu_bwd(
                P(b[2]), None, None, P(b[1]), P(b[0]), P(bias), rows, cols, BF16, st))), n, 3)
            res.append(roof(f"bias_gelu_bwd without dbias {shape}", 6 * n_el, t, n_el, n_sets))
            t = time_launches(rotating(sets, lambda b: check(lib.oslo_bias_dropout_add_bwd(
                P(b[2]), None, None, P(b[1]), 0.1, 1234, 0, rows, cols, BF16, st))), n, 3)
            res.append(roof(f"bias_dropout_add_bwd without dbias p=0.1 {shape}", 4 * n_el, t, n_el, n_sets))
            # the same two backward kernels on one set of buffers: what a consumer sees whose input the
            # kernel before it has just written (a good part of it is still in the 256 MB memory-side cache)
            b = sets[0]
            t = time_launches(lambda: check(lib.oslo_bias_gelu_bwd(
                P(b[2]), P(db), P(ws), P(b[1]), P(b[0]), P(bias), rows, cols, BF16, st)), n, 3)
            res.append(roof(f"bias_gelu_bwd+dbias {shape} (same buffers every launch)", 6 * n_el, t, n_el, 1))
            t = time_launches(lambda: check(lib.oslo_bias_dropout_add_bwd(
                P(b[2]), P(db), P(ws), P(b[1]), 0.1, 1234, 0, rows, cols, BF16, st)), n, 3)
            res.append(roof(f"bias_dropout_add_bwd+dbias p=0.1 {shape} (same buffers every launch)", 4 * n_el, t, n_el, 1))
        del sets, ws

    # rotary embedding + split heads of q, k, v at the GPT-J-6B shape
    B, S, H, D, rot = 8, 2048, 16, 256, 64
    sets = [tuple(randn((B, S, H, D), 10 + 3 * j + i, 1.0, torch.bfloat16) for i in range(3)) +
            tuple(torch.empty((B, H, S, D), dtype=torch.bfloat16, device=dev) for _ in range(3)) for j in range(4)]
    from oslo_amd.modeling_gptj import rotary_tables
    sin, cos = rotary_tables(rot, S, dev)
    t = time_launches(rotating(sets, lambda b: check(lib.oslo_rotary_qkv(
        P(b[3]), P(b[4]), P(b[5]), P(b[0]), P(b[1]), P(b[2]), P(sin), P(cos),
        S, B, S, H, D, 0, rot, 0, 0, BF16, st))), n, 3)
    n_el = B * S * H * D
    res.append(roof("rotary_qkv bf16 q,k,v [8,2048,16,256] rotary 64", 3 * 4 * n_el, t, 3 * n_el, len(sets)))
    del sets

    # the projections of a decoding step at the GPT-J-6B shape: the weight is the traffic
    for n_out, k_in, gelu, what in ((16384, 4096, 1, "fc_in + bias + gelu"), (4096, 16384, 0, "fc_out + bias"),
                                    (4096, 4096, 0, "attention projection")):
        n_sets = max(2, (1 << 30) // (n_out * k_in * 2))
        weights = [randn((n_out, k_in), 20 + i, 0.02, torch.bfloat16) for i in range(n_sets)]
        bias = randn((n_out,), 4, 0.02, torch.bfloat16)
        for m in (1, 8):
            xin = randn((m, k_in), 5, 1.0, torch.bfloat16)
            o = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
            t = time_launches(rotating(weights, lambda wt: check(lib.oslo_linear_rows_fwd(
                P(o), P(xin), P(wt), P(bias), None, m, n_out, k_in, gelu, BF16, st))), n, 3)
            res.append(roof(f"linear_rows {what} bf16 {m} x [{n_out},{k_in}]",
                            2 * (n_out * k_in + m * k_in + m * n_out + n_out), t, m * n_out, n_sets))
        del weights

    # the attention of a decoding step at the GPT-J head shape: 1024 visible keys of a 1152-slot cache
    H, cap, D, last = 16, 1152, 256, 1023
    for rows in (1, 8):
        n_sets = 8
        caches = [(randn((rows * H, cap, D), 30 + i, 1.0, torch.bfloat16), randn((rows * H, cap, D), 40 + i, 1.0, torch.bfloat16))
                  for i in range(n_sets)]
        qd = randn((rows * H, D), 6, 1.0, torch.bfloat16)
        od = torch.empty_like(qd)
        wsd = torch.empty(lib.oslo_attention_decode_workspace_bytes(rows * H, cap, D, BF16) // 4,
                          dtype=torch.float32, device=dev)
        t = time_launches(rotating(caches, lambda kv: check(lib.oslo_attention_decode_fwd(
            P(od), P(qd), P(kv[0]), P(kv[1]), None, None, 0, 0, P(wsd), None, last, 0, 1 / 16.0, rows * H, cap, D, BF16, st))), n, 3)
        res.append(roof(f"attention_decode bf16 {rows} x 16 heads, 1024 of 1152 keys, head 256 (two launches)",
                        2 * 2 * rows * H * (last + 1) * D, t, rows * H * D, n_sets))
        del caches

    # Calibration of the matrix-core rows below: the library's dense bf16 GEMM, 8192^3, unit-normal operands,
    # in this process and clock state. What it sustains is what a kernel made of nothing but matrix
    # products reaches on this part against the published peak.
    ga, gb = randn((8192, 8192), 70, 1.0, torch.bfloat16), randn((8192, 8192), 71, 1.0, torch.bfloat16)
    gc = torch.empty_like(ga)
    t = time_launches(lambda: torch.matmul(ga, gb, out=gc), max(5, n // 4), 3)
    gflops = 2 * 8192 ** 3
    res.append({"kernel": "torch.matmul bf16 8192 x 8192 x 8192 (calibration, not a kernel of this library)",
                "bound": "mfma", "achieved": round(gflops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(gflops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                "us": round(t * 1e6, 1), "algorithmic_flops": gflops, "traffic": None})
    ga.zero_(), gb.zero_()
    t = time_launches(lambda: torch.matmul(ga, gb, out=gc), max(5, n // 4), 3)
    res.append({"kernel": "torch.matmul bf16 8192 x 8192 x 8192, zero operands (calibration)",
                "bound": "mfma", "achieved": round(gflops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(gflops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                "us": round(t * 1e6, 1), "algorithmic_flops": gflops, "traffic": None})
    del ga, gb, gc

    # causal attention over a whole prompt in one kernel, at the GPT-J shape and a GPT-Neo-sized one:
    # the one kernel here that is bound by the matrix cores (4 flops per score and feature, lower triangle)
    import ctypes
    for (B, Hh, S, D) in ((8, 16, 2048, 256), (8, 16, 2048, 128), (1, 16, 8192, 256)):
        q, k, v = (randn((B, Hh, S, D), 50 + i, 1.0, torch.bfloat16) for i in range(3))
        o = torch.empty((B, S, Hh, D), dtype=torch.bfloat16, device=dev)
        strides = (ctypes.c_int64 * 12)(*(3 * [Hh * S * D, S * D, D] + [S * Hh * D, D, Hh * D]))
        flops = 4 * B * Hh * D * (S * (S + 1) // 2)
        lens = torch.randint(S // 2, S + 1, (B,), device=dev, generator=torch.Generator(device=dev).manual_seed(2))
        key_pad = torch.where(torch.arange(S, device=dev)[None, :] < lens[:, None], 0.0, -10000.0).float().contiguous()
        for what, mask in (("causal", None), ("causal with padding mask", key_pad)):
            if mask is not None and (D != 256 or S != 2048):
                continue
            t = time_launches(lambda: check(lib.oslo_attention_prefill_fwd(
                P(o), P(q), P(k), P(v), P(mask) if mask is not None else None, D ** -0.5, B, Hh, S, D, 0, strides,
                BF16, st)), max(5, n // 2), 3)
            res.append({"kernel": f"attention_prefill bf16 [{B},{Hh},{S},{D}] {what}", "bound": "mfma",
                        "achieved": round(flops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4), "us": round(t * 1e6, 1),
                        "algorithmic_flops": flops, "traffic": None})
        if S != 2048:  # the long prompt: forward only
            del q, k, v, o
            continue
        # its backward (the forward that stores the log-sum-exp first). Algorithmic work: the five
        # matrix products of the mathematics (S, dP, dV, dQ, dK) where the forward has two, 10 flops per
        # visible score and feature; `frac` is that over the time. Where each owner kind recomputes the
        # scores the kernels issue more (`issued_flops`: BWD_PRODUCTS_ISSUED products per visible tile).
        lse = torch.empty((B, Hh, S), dtype=torch.float32, device=dev)
        check(lib.oslo_attention_prefill_fwd_lse(P(o), P(lse), P(q), P(k), P(v), None, D ** -0.5, 0.0, 0, 0,
                                                 B, Hh, S, D, 0, strides, BF16, st))
        do = randn((B, S, Hh, D), 60, 1.0, torch.bfloat16)
        dq, dk, dv = (torch.empty((B, Hh, S, D), dtype=torch.bfloat16, device=dev) for _ in range(3))
        wsb = torch.empty(lib.oslo_attention_prefill_bwd_workspace_bytes(B, Hh, S) // 4, dtype=torch.float32, device=dev)
        dense, merged = [Hh * S * D, S * D, D], [S * Hh * D, D, Hh * D]
        bstr = (ctypes.c_int64 * 24)(*(3 * dense + 2 * merged + 3 * dense))
        recompute = lambda: check(lib.oslo_attention_prefill_bwd(
            P(dq), P(dk), P(dv), P(do), P(q), P(k), P(v), P(o), P(lse), P(wsb), None, D ** -0.5, 0.0, 0, 0,
            B, Hh, S, D, 0, bstr, BF16, st))
        backward = recompute
        bflops = 5 * flops // 2
        if D == 256:
            # what the operator runs at this head size: the dQ pass hands P and dS to the dK/dV pass
            # through a tile store (16-bit, the tiles on and below the diagonal), 5 products per tile
            store_bytes = lib.oslo_attention_prefill_bwd_store_bytes(B, Hh, S)
            store = torch.empty(store_bytes, dtype=torch.uint8, device=dev)
            backward = lambda: check(lib.oslo_attention_prefill_bwd_stored(
                P(dq), P(dk), P(dv), P(do), P(q), P(k), P(v), P(o), P(lse), P(wsb), P(store), store_bytes, None,
                D ** -0.5, 0.0, 0, 0, B, Hh, S, D, 0, bstr, BF16, st))
            t = time_launches(recompute, max(5, n // 4), 3)
            issued = BWD_PRODUCTS_ISSUED[D] * flops // 2
            res.append({"kernel": f"attention_prefill_bwd bf16 [{B},{Hh},{S},{D}] causal, every pass computing its "
                                  "scores (no tile store)", "bound": "mfma",
                        "achieved": round(bflops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(bflops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4), "us": round(t * 1e6, 1),
                        "algorithmic_flops": bflops, "issued_flops": issued,
                        "issued_TFLOPs": round(issued / t / 1e12, 1), "traffic": None})
        t = time_launches(backward, max(5, n // 4), 3)
        issued = (5 if D == 256 else BWD_PRODUCTS_ISSUED[D]) * flops // 2
        row = {"kernel": f"attention_prefill_bwd bf16 [{B},{Hh},{S},{D}] causal (dq, dk, dv)",
               "bound": "mfma",
               "achieved": round(bflops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
               "frac": round(bflops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4), "us": round(t * 1e6, 1),
               "algorithmic_flops": bflops, "issued_flops": issued,
               "issued_TFLOPs": round(issued / t / 1e12, 1), "traffic": None}
        if D == 256:
            row["tile_store_bytes"] = store_bytes
        res.append(row)
        if D == 256:
            # The same launches on zero operands: the same instructions in the same order (no branch of
            # these kernels looks at the data), without the switching activity of the matrix cores'
            # inputs. The gap to the rows above is the clock the chip sustains under that activity, not
            # something the kernels' code decides.
            for x in (q, k, v, do):
                x.zero_()
            t = time_launches(lambda: check(lib.oslo_attention_prefill_fwd(
                P(o), P(q), P(k), P(v), None, D ** -0.5, B, Hh, S, D, 0, strides, BF16, st)), max(5, n // 2), 3)
            res.append({"kernel": f"attention_prefill bf16 [{B},{Hh},{S},{D}] causal, zero operands (same instruction stream)",
                        "bound": "mfma", "achieved": round(flops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                        "us": round(t * 1e6, 1), "algorithmic_flops": flops, "traffic": None})
            check(lib.oslo_attention_prefill_fwd_lse(P(o), P(lse), P(q), P(k), P(v), None, D ** -0.5, 0.0, 0, 0,
                                                     B, Hh, S, D, 0, strides, BF16, st))
            t = time_launches(backward, max(5, n // 4), 3)
            res.append({"kernel": f"attention_prefill_bwd bf16 [{B},{Hh},{S},{D}] causal, zero operands (same instruction stream)",
                        "bound": "mfma", "achieved": round(bflops / t / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(bflops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                        "us": round(t * 1e6, 1), "algorithmic_flops": bflops, "issued_flops": issued,
                        "issued_TFLOPs": round(issued / t / 1e12, 1), "traffic": None})
        del q, k, v, o, do, dq, dk, dv, lse, wsb
        if D == 256:
            del store
    return res


def run_only(args, lib, torch, dev, st, P, check, time_launches, fwd, bwd):
    """--only causal_fwd | causal_bwd | attention_prefill | attention_prefill_bwd | gemm | copy: launch one kernel
    (the backward: its four) `steps` times
    (profiling runs). `copy` is torch's device copy of 1 GiB, the kernel of
    known traffic that calibrates the FETCH_SIZE / WRITE_SIZE counters."""
    if args.only.startswith("gptj_"):
        model_pass_only(args, torch, dev)
        return
    if args.only == "copy":
        a = torch.ones(1 << 30, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        fn = lambda: b.copy_(a)
    elif args.only == "gemm":
        # the calibration of the matrix-core rows: the library's dense bf16 GEMM, 8192^3
        ga, gb = (torch.randn(8192, 8192, device=dev).to(torch.bfloat16) for _ in range(2))
        if args.zero_operands:
            ga.zero_(), gb.zero_()
        gc = torch.empty_like(ga)
        fn = lambda: torch.matmul(ga, gb, out=gc)
    elif args.only in ("attention_prefill_bwd", "attention_prefill_bwd_recompute"):
        import ctypes
        B, Hh, S, D = 8, 16, 2048, 256  # the GPT-J shape of the kernel table
        q, k, v, do = (torch.randn(B, Hh, S, D, device=dev).to(torch.bfloat16) for _ in range(4))
        o = torch.empty((B, Hh, S, D), dtype=torch.bfloat16, device=dev)
        lse = torch.empty((B, Hh, S), dtype=torch.float32, device=dev)
        dense = [Hh * S * D, S * D, D]
        check(lib.oslo_attention_prefill_fwd_lse(P(o), P(lse), P(q), P(k), P(v), None, D ** -0.5, 0.0, 0, 0,
                                                 B, Hh, S, D, 0, (ctypes.c_int64 * 12)(*(4 * dense)), 2, st))
        dq, dk, dv = (torch.empty_like(q) for _ in range(3))
        ws = torch.empty(lib.oslo_attention_prefill_bwd_workspace_bytes(B, Hh, S) // 4, dtype=torch.float32, device=dev)
        bstr = (ctypes.c_int64 * 24)(*(8 * dense))
        if args.only.endswith("_recompute"):  # every pass computes its scores: nothing of [S, S] in memory
            fn = lambda: check(lib.oslo_attention_prefill_bwd(
                P(dq), P(dk), P(dv), P(do), P(q), P(k), P(v), P(o), P(lse), P(ws), None, D ** -0.5, 0.0, 0, 0,
                B, Hh, S, D, 0, bstr, 2, st))
        else:  # what the operator runs at this head size: P and dS handed to the dK/dV pass through a tile store
            store_bytes = lib.oslo_attention_prefill_bwd_store_bytes(B, Hh, S)
            store = torch.empty(store_bytes, dtype=torch.uint8, device=dev)
            fn = lambda: check(lib.oslo_attention_prefill_bwd_stored(
                P(dq), P(dk), P(dv), P(do), P(q), P(k), P(v), P(o), P(lse), P(ws), P(store), store_bytes, None,
                D ** -0.5, 0.0, 0, 0, B, Hh, S, D, 0, bstr, 2, st))
    elif args.only == "attention_prefill":
        import ctypes
        B, Hh, S, D = 8, 16, 2048, 256  # the GPT-J shape of the kernel table
        q, k, v = (torch.randn(B, Hh, S, D, device=dev).to(torch.bfloat16) for _ in range(3))
        if args.zero_operands:  # the same instruction stream without the switching activity of its inputs
            for x in (q, k, v):
                x.zero_()
        o = torch.empty((B, S, Hh, D), dtype=torch.bfloat16, device=dev)
        strides = (ctypes.c_int64 * 12)(*(3 * [Hh * S * D, S * D, D] + [S * Hh * D, D, Hh * D]))
        fn = lambda: check(lib.oslo_attention_prefill_fwd(
            P(o), P(q), P(k), P(v), None, D ** -0.5, B, Hh, S, D, 0, strides, 2, st))
    else:
        fn = {"causal_fwd": fwd, "causal_bwd": bwd}.get(args.only)
    if fn is None:
        sys.exit("--only takes causal_fwd, causal_bwd, attention_prefill, attention_prefill_bwd, "
                 "attention_prefill_bwd_recompute, gemm, copy or a gptj_* pass")
    if args.only == "causal_bwd":
        fwd()
    t = time_launches(fn, args.steps, args.warmup)
    print(json.dumps({"only": args.only, "us": round(t * 1e6, 2), "launches": args.steps}))


def model_pass_only(args, torch, dev):
    """--only gptj_fwd_fused | gptj_fwd_unfused: `steps` forward passes of the
    GPT-J-6B-shaped model of the `gptj_fwd` section (28 layers, batch 8 x 2048,
    eval), after fuse() or before it; --only gptj_train_fused |
    gptj_train_unfused: `steps` forward + backward passes of the 4-layer stack
    of the `gptj_train_step` section (attention and residual dropout 0.1).
    Nothing else runs: a kernel trace of the command is the model's kernel mix."""
    from oslo_amd import GPTJConfig, GPTJForCausalLM

    what, fused = args.only.rsplit("_", 1)
    if what not in ("gptj_fwd", "gptj_train") or fused not in ("fused", "unfused"):
        sys.exit("--only takes gptj_fwd_fused, gptj_fwd_unfused, gptj_train_fused or gptj_train_unfused")
    train = what == "gptj_train"
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            torch.manual_seed(0)
            cfg = GPTJConfig(n_layer=4, attn_pdrop=0.1, resid_pdrop=0.1) if train else GPTJConfig(n_layer=28)
            model = GPTJForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    model = model.train() if train else model.eval()
    if fused == "fused":
        model.fuse()
    ids = torch.randint(0, 50400, (8, 2048), device=dev)

    def run():
        if train:
            model.zero_grad(set_to_none=True)
            model(ids, labels=ids)["loss"].backward()
        else:
            with torch.no_grad():
                model(ids)

    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    print(json.dumps({"only": args.only, "ms": round(ms, 2), "tokens_per_s": round(8 * 2048 / ms * 1e3, 1),
                      "passes": args.steps}))


def gptj_forward(torch, dev, layers=28, batch=8, seq=2048, reps=5):
    """GPT-J-6B-shaped forward (28 layers, d_model 4096, 16 heads of 256, rotary
    64, d_ff 16384, vocab 50400; weights N(0, 0.02) in bf16; token ids uniform;
    eval mode), unfused torch modules against the same model after fuse()."""
    from oslo_amd import GPTJConfig, GPTJForCausalLM

    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            torch.manual_seed(0)
            model = GPTJForCausalLM(GPTJConfig(n_layer=layers)).eval()
    finally:
        torch.set_default_dtype(old)
    ids = torch.randint(0, 50400, (batch, seq), device=dev)

    def run():
        with torch.no_grad():
            return model(ids)["logits"]

    def timed():
        for _ in range(2):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    def decode_ms(context=1024, steps=20):
        """One new token for one sequence over a key/value cache of `context`
        tokens: milliseconds per step (bound by launches, not by the kernels)."""
        with torch.no_grad():
            past = model(ids[:1, :context], use_cache=True)["past_key_values"]
            nxt = ids[:1, context - 1:context]
            for _ in range(3):
                model(nxt, past_key_values=past, use_cache=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                model(nxt, past_key_values=past, use_cache=True)
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    def graphed_decode_ms(context=1024, steps=20):
        """The same step over preallocated caches, replayed as one HIP graph."""
        from oslo_amd.generation_utils import StaticDecoder

        with torch.no_grad():
            decoder = StaticDecoder(model, context + steps + 8, graph=True)
            seq_ids = ids[:1, :context]
            decoder.step(seq_ids)
            for n in range(3):  # the first of these captures
                seq_ids = torch.cat([seq_ids, ids[:1, n:n + 1]], dim=1)
                decoder.step(seq_ids)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for n in range(steps):
                seq_ids = torch.cat([seq_ids, ids[:1, n:n + 1]], dim=1)
                decoder.step(seq_ids)
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    # Parity of the timed model, at all its layers: the same weights in fp32, unfused, on the first two
    # sequences are the yardstick; the fused bf16 logits must be no further from them than the unfused
    # bf16 logits are (their mutual difference is then where the 16-bit roundings fall, not an error).
    import copy
    with torch.no_grad():
        ref32 = copy.deepcopy(model).float()(ids[:2])["logits"]
    torch.cuda.empty_cache()
    t_unfused = timed()
    with torch.no_grad():
        unfused2 = model(ids[:2])["logits"].float()
    d_unfused = decode_ms()
    model.fuse()
    t_fused = timed()
    with torch.no_grad():
        fused2 = model(ids[:2])["logits"].float()
    err_u, err_f = (unfused2 - ref32).abs(), (fused2 - ref32).abs()
    top = ref32.argmax(-1)
    vs_fp32 = {"sequences": 2, "unfused_mean_abs": round(err_u.mean().item(), 6), "fused_mean_abs": round(err_f.mean().item(), 6),
               "unfused_max_abs": round(err_u.max().item(), 4), "fused_max_abs": round(err_f.max().item(), 4),
               "fused_vs_unfused_max_abs": round((fused2 - unfused2).abs().max().item(), 4),
               "unfused_top1_agreement": round((unfused2.argmax(-1) == top).float().mean().item(), 4),
               "fused_top1_agreement": round((fused2.argmax(-1) == top).float().mean().item(), 4)}
    del ref32, unfused2, fused2, err_u, err_f
    if not (vs_fp32["fused_mean_abs"] <= 1.05 * vs_fp32["unfused_mean_abs"]
            and vs_fp32["fused_max_abs"] <= 1.25 * vs_fp32["unfused_max_abs"]):
        raise AssertionError(f"fused logits are further from the fp32 model than the unfused bf16 logits: {vs_fp32}")
    d_fused = decode_ms()
    d_graph = graphed_decode_ms()
    del model
    torch.cuda.empty_cache()
    tokens = batch * seq
    return {"config": f"{layers} layers, d_model 4096, 16x256 heads, rotary 64, d_ff 16384, vocab 50400, "
                      f"bf16, batch {batch}, seq {seq}, eval",
            "unfused_tokens_per_s": round(tokens / t_unfused, 1), "fused_tokens_per_s": round(tokens / t_fused, 1),
            "unfused_ms": round(t_unfused * 1e3, 2), "fused_ms": round(t_fused * 1e3, 2),
            "speedup": round(t_unfused / t_fused, 3), "logits_vs_fp32": vs_fp32,
            "decode_step_batch1_context1024": {"unfused_ms": round(d_unfused, 2), "fused_ms": round(d_fused, 2),
                                               "speedup": round(d_unfused / d_fused, 3),
                                               "fused_graph_replay_ms": round(d_graph, 2)}}


def gptj_train_step(torch, dev, attn_pdrop=0.1, layers=4, batch=8, seq=2048, reps=3):
    """Forward + backward (loss on the input ids, no optimizer) of a GPT-J-6B-
    shaped stack cut to `layers` layers, with attention and residual dropout at
    0.1, unfused torch modules against the same model after fuse(): the
    backward kernels and the dropout kernels in place."""
    from oslo_amd import GPTJConfig, GPTJForCausalLM

    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            torch.manual_seed(0)
            model = GPTJForCausalLM(GPTJConfig(n_layer=layers, attn_pdrop=attn_pdrop, resid_pdrop=0.1)).train()
    finally:
        torch.set_default_dtype(old)
    ids = torch.randint(0, 50400, (batch, seq), device=dev)

    def run():
        model.zero_grad(set_to_none=True)
        loss = model(ids, labels=ids)["loss"]
        loss.backward()
        return loss

    def timed():
        for _ in range(2):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    t_unfused = timed()
    torch.cuda.reset_peak_memory_stats(dev)
    run()
    mem_unfused = torch.cuda.max_memory_allocated(dev)
    model.fuse()
    t_fused = timed()
    torch.cuda.reset_peak_memory_stats(dev)
    loss = run()
    mem_fused = torch.cuda.max_memory_allocated(dev)
    finite = bool(torch.isfinite(loss).item())
    del model
    torch.cuda.empty_cache()
    tokens = batch * seq
    return {"config": f"{layers} layers of the 6B shape, bf16, batch {batch}, seq {seq}, attention dropout "
                      f"{attn_pdrop}, residual dropout 0.1, forward + backward",
            "unfused_tokens_per_s": round(tokens / t_unfused, 1), "fused_tokens_per_s": round(tokens / t_fused, 1),
            "unfused_ms": round(t_unfused * 1e3, 2), "fused_ms": round(t_fused * 1e3, 2),
            "speedup": round(t_unfused / t_fused, 3),
            "unfused_peak_GiB": round(mem_unfused / 2 ** 30, 2), "fused_peak_GiB": round(mem_fused / 2 ** 30, 2),
            "loss_finite": finite}


def other_families_forward(torch, dev, reps=5):
    """fuse() on the two other model families of the path, forward in eval mode,
    at published shapes cut to a few layers: GPT-2 XL blocks (d_model 1600, 25
    heads of 64, 1024 positions) in fp16 and GPT-Neo 2.7B blocks (d_model 2560,
    20 heads of 128, 2048 positions; every second layer is a sliding-window
    layer) in fp16, the one dtype the reference's gate admits. GPT-Neo does
    not scale its scores; with random N(0, 0.02) weights at this width they
    have a standard deviation of about 11, so its softmax is close to a
    maximum and amplifies the 16-bit roundings that the fused and the unfused
    modules make at different places (bias and GeLU on fp32 sums against one
    rounding per operator): the logit difference reported for this family is
    that sensitivity, not the kernels (in fp32 the two paths agree to 2e-4)."""
    from oslo_amd import GPT2Config, GPT2LMHeadModel, GPTNeoConfig, GPTNeoForCausalLM

    cases = [
        ("gpt2_xl_blocks", torch.float16, 16, 1024,
         lambda: GPT2LMHeadModel(GPT2Config(n_embd=1600, n_head=25, n_layer=6, n_positions=1024))),
        ("gpt_neo_2.7b_blocks", torch.float16, 8, 2048,
         lambda: GPTNeoForCausalLM(GPTNeoConfig(hidden_size=2560, num_heads=20, num_layers=6,
                                                max_position_embeddings=2048))),
    ]
    res = {}
    for name, dtype, batch, seq, ctor in cases:
        old = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            with torch.device(dev):
                torch.manual_seed(0)
                model = ctor().eval()
        finally:
            torch.set_default_dtype(old)
        ids = torch.randint(0, 50257, (batch, seq), device=dev)

        def run():
            with torch.no_grad():
                return model(ids)["logits"]

        def timed():
            for _ in range(2):
                run()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                run()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / reps

        t_unfused = timed()
        ref_logits = run().float()
        model.fuse()
        t_fused = timed()
        diff = (run().float() - ref_logits).abs().max().item()
        del model, ref_logits
        torch.cuda.empty_cache()
        res[name] = {"dtype": str(dtype).replace("torch.", ""), "batch": batch, "seq": seq, "layers": 6,
                     "unfused_tokens_per_s": round(batch * seq / t_unfused, 1),
                     "fused_tokens_per_s": round(batch * seq / t_fused, 1),
                     "speedup": round(t_unfused / t_fused, 3), "max_abs_logit_diff": round(diff, 4)}
    return res


def cpu_baseline(torch, section=lambda fn, *a: fn(*a)):
    """The unfused arithmetic with torch's CPU operators on the host cores, fp32
    (CPU half softmax is not representative), on bounded samples of the same
    workloads, best of 5 passes each: the causal softmax forward + autograd
    backward on [1,4,2048,2048] slabs (the figure of `value`), gelu_new(x + b)
    and dropout(x + b) + residual on [2048,4096] bands. The thread count is set
    explicitly to the cores this process may use and reported."""
    from oracle import unfused_torch as ref

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():  # the share of the machine this job was given
        cores = min(cores, int(os.environ["OMP_NUM_THREADS"]))
    torch.set_num_threads(cores)
    cores = torch.get_num_threads()
    b, h, s = 1, 4, 2048
    gen = torch.Generator().manual_seed(0)
    x = torch.randn((b, h, s, s), generator=gen) * 8
    go = torch.randn((b, h, s, s), generator=gen)
    tri, full = b * h * s * (s + 1) // 2, b * h * s * s
    # same accounting as the GPU figure, at the fp16 element size of the workload
    nbytes = 2 * (tri + full) + 2 * (2 * tri + full)

    def best_of(fn, passes=5, budget=4.0):
        fn()
        best, t_start = float("inf"), time.perf_counter()
        for i in range(passes):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
            if time.perf_counter() - t_start > budget and i >= 1:
                break
        return best

    def softmax_step():
        xx = x.clone().requires_grad_(True)
        y = ref.attention_probs(xx, 0.125, causal=True)
        y.backward(go)

    dt = best_of(softmax_step, budget=10.0)
    rows, cols = 2048, 4096
    a = torch.randn((rows, cols), generator=gen)
    r = torch.randn((rows, cols), generator=gen)
    bias = torch.randn((cols,), generator=gen) * 0.02
    n_el = rows * cols
    t_gelu = best_of(lambda: ref.bias_gelu(a, bias))
    torch.manual_seed(1234)
    t_drop = best_of(lambda: ref.bias_dropout_add(a, bias, r, 0.1, True))
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"unfused fp32 causal softmax fwd+bwd on [1,4,2048,2048], best of 5: "
                      f"{dt * 1e3:.1f} ms, bytes counted at the workload's fp16 size",
            "bias_gelu_fwd_GBps": round(4 * n_el / t_gelu / 1e9, 3),
            "bias_dropout_add_fwd_GBps": round(6 * n_el / t_drop / 1e9, 3),
            "elementwise_sample": f"gelu_new(x + b) and dropout(x + b, 0.1) + residual on fp32 [{rows},{cols}], "
                                  "best of 5, bytes counted at the bf16 size of the GPU rows (4 and 6 B per element)",
            "gpt2_small_fwd": section(gpt2_small_forward, torch),
            "gpt2_small_generate": section(gpt2_small_generate, torch)}


def gpt2_small_generate(torch):
    """The reference's kernel-fusion test (tests/gpt2/gpt2_test_kernel_fusion.py:
    26-49) on random weights: GPT-2 small, fp32, one prompt of 12 tokens, beam
    search with 5 beams to exactly 200 tokens, no 4-gram twice. Seconds per
    generate() before fuse(), after it, with the fused n-gram ban, and with each
    step replayed as a HIP graph (capture included)."""
    from oslo_amd import GPT2Config, GPT2LMHeadModel

    torch.manual_seed(0)
    model = GPT2LMHeadModel(GPT2Config(resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)).eval().to("cuda:0")
    ids = torch.randint(0, 50257, (1, 12), generator=torch.Generator().manual_seed(1)).to("cuda:0")
    kw = dict(max_length=200, min_length=200, num_beams=5, no_repeat_ngram_size=4)

    def run(**extra):
        for _ in range(2):
            model.generate(ids, **kw, **extra)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = model.generate(ids, **kw, **extra)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, out

    t_before, want = run()
    model = model.fuse()
    t_after, out_after = run()
    t_ban, out_ban = run(fused_no_repeat_ngram_blocking=True)
    t_graph, out_graph = run(fused_no_repeat_ngram_blocking=True, graph=True)
    return {"config": "GPT-2 small fp32 random weights, prompt 12 tokens, max_length=min_length=200, num_beams=5, "
                      "no_repeat_ngram_size=4",
            "before_fuse_s": round(t_before, 3), "after_fuse_s": round(t_after, 3),
            "after_fuse_fused_ngram_ban_s": round(t_ban, 3), "after_fuse_graph_replay_s": round(t_graph, 3),
            "same_tokens": bool(torch.equal(want, out_after) and torch.equal(want, out_ban)
                                and torch.equal(want, out_graph))}


def gpt2_small_forward(torch):
    """The CPU-runnable configuration: GPT-2 small (12 layers, d_model 768, 12
    heads, vocab 50257), random fp32 weights, batch 4 x 512 tokens, eval. The
    unfused model on the host cores against the same weights after fuse() on
    the GPU."""
    from oslo_amd import GPT2Config, GPT2LMHeadModel

    torch.manual_seed(0)
    model = GPT2LMHeadModel(GPT2Config()).eval()
    ids = torch.randint(0, 50257, (4, 512))
    with torch.no_grad():
        model(ids)
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 5.0 or reps < 2:
            cpu_logits = model(ids)["logits"]
            reps += 1
        t_cpu = (time.perf_counter() - t0) / reps
        model = model.to("cuda:0").fuse()
        dev_ids = ids.to("cuda:0")
        for _ in range(3):
            gpu_logits = model(dev_ids)["logits"]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            model(dev_ids)
        torch.cuda.synchronize()
        t_gpu = (time.perf_counter() - t0) / 20
        # the same forward captured once as a HIP graph and replayed
        from oslo_amd import GraphedForward
        graphed = GraphedForward(model, dev_ids)
        for _ in range(3):
            graph_logits = graphed(dev_ids)["logits"]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            graphed(dev_ids)
        torch.cuda.synchronize()
        t_graph = (time.perf_counter() - t0) / 20
    diff = (gpu_logits.cpu() - cpu_logits).abs().max().item()
    return {"cpu_unfused_tokens_per_s": round(2048 / t_cpu, 1), "cpu_cores": torch.get_num_threads(),
            "gpu_fused_tokens_per_s": round(2048 / t_gpu, 1),
            "gpu_fused_graph_replay_tokens_per_s": round(2048 / t_graph, 1),
            "graph_equals_eager": bool(torch.equal(graph_logits, gpu_logits)),
            "max_abs_logit_diff": round(diff, 6)}


if __name__ == "__main__":
    main()
