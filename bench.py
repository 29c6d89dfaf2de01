#!/usr/bin/env python3
"""Benchmark of the cosine-linear-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A step is one causal forward + backward (dQ, dK, dV) over one synthetic batch at the headline
shape B=8 H=16 N=2048 D=64 bf16, called through the C ABI on torch's current stream with every
input already resident in HBM, the way CustomAttention runs it: the forward also leaves one 16 KiB
state per head that the backward starts dQ from (the plain entry points are timed beside it).  Prints ONE JSON line: whole-job tokens/s, the roofline object of
the dominant kernel (HIP events recorded by the library around each of its launches), and the CPU
baseline (the reference's PyTorch cumsum formulation timed on the host cores of this box).
"""
import argparse
import json
import os
import statistics
import sys
import time

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
SPINUP_S = 0.3               # untimed GPU spin-up before the warm-up steps
MFMA_BF16_PEAK_TFLOPS = 2500.0

# HBM-side bytes per launch at the headline shape, from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs of
# `bench.py --calibration-copy` (counters scaled by their reading for the 256 MiB copy in the same run).
# A counter run cannot be made from inside this script; the figures and commands are in
# profiles/headline_kernels_hbm_traffic_pmc.txt.
MEASURED_TRAFFIC_BYTES = {"scan": 127.19 * 2**20, "scan_grad": 223.05 * 2**20}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary configs (non-causal, decode, long)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--block-only", action="store_true",
                    help="run only the GPT attention block fwd+bwd (a secondary figure) for --steps steps: for profiling")
    ap.add_argument("--bert-block-only", action="store_true",
                    help="run only the BERT self-attention block fwd+bwd (a secondary figure) for --steps steps: for profiling")
    ap.add_argument("--long-only", type=int, default=0, metavar="N",
                    help="run only the long-context configuration B1 H16 D128 bf16 at sequence length N (fwd and bwd "
                         "separately, per-kernel durations) for --steps steps: for profiling")
    ap.add_argument("--cold-only", action="store_true",
                    help="run only the headline forward and gradient launches with cold caches (and the streaming-only "
                         "kernel of their launch shape): for counter runs whose per-dispatch averages are cold launches")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device copy (a kernel of known traffic, to scale rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


def make_inputs(torch, b, h, n, dk, dv, dtype, device, seed=0, grad=True):
    g = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(b, h, n, dk, generator=g), p=2, dim=-1)
    k = torch.nn.functional.normalize(torch.randn(b, h, n, dk, generator=g), p=2, dim=-1)
    v = torch.randn(b, h, n, dv, generator=g)
    out = [q, k, v]
    if grad:
        out.append(torch.randn(b, h, n, dv, generator=g))
    return [t.to(dtype).to(device) for t in out]


def time_region(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def cpu_baseline(torch):
    """Reference CPU path: cumsum form forward (GPT_Trainer/GPTCosAttention.py:319) + autograd
    backward, fp32, on a bounded sample: one batch element of the headline shape."""
    from oracle import torch_forms as tf
    b, h, n, d = 1, 16, 2048, 64
    q, k, v, g = tf.synthetic_inputs((b, h, n, d), seed=0, dtype=torch.float32)
    times = []
    for it in range(25):
        qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
        t0 = time.perf_counter()
        tf.causal_cumsum(qa, ka, va).backward(g)
        times.append(time.perf_counter() - t0)
    t = statistics.median(times[1:])
    # the reference's own CPU-runnable configuration, (1,2,128,64) fp32, same formulation
    q1, k1, v1, g1 = tf.synthetic_inputs((1, 2, 128, 64), seed=0, dtype=torch.float32)
    t1s = []
    for it in range(23):
        qa, ka, va = (x.clone().requires_grad_(True) for x in (q1, k1, v1))
        t0 = time.perf_counter()
        tf.causal_cumsum(qa, ka, va).backward(g1)
        t1s.append(time.perf_counter() - t0)
    t1 = statistics.median(t1s[3:])
    return {"value": b * n / t, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"(B,H,N,D)=({b},{h},{n},{d}) fp32: 1 of the 8 batch elements of the headline shape, torch cumsum "
                      f"form fwd + autograd bwd, median of 24 passes after 1 warm-up; {t:.2f} s per pass",
            "cfg1_B1_H2_N128_D64_fp32": {"value": 128 / t1, "unit": "tokens/s", "ms_per_pass": t1 * 1e3,
                                         "sample": "median of 20 passes after 3 warm-ups"}}


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    import cottention_transformer_amd as ct
    from cottention_transformer_amd import _loader

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.block_only:
        block_step = gpt_block_step(torch, dev)
        s = time_region(torch, lambda: block_step(False), args.steps, args.warmup)
        print(json.dumps({"gpt_block_fwd_bwd_B8_S2048_E1024_H16_autocast_bf16_us": s * 1e6, "steps": args.steps,
                          "warmup": args.warmup}))
        return
    if args.bert_block_only:
        step = bert_block_step(torch, dev)
        s = time_region(torch, step, args.steps, args.warmup)
        print(json.dumps({"bert_block_fwd_bwd_B32_S512_E768_H12_autocast_bf16_us": s * 1e6, "steps": args.steps,
                          "warmup": args.warmup}))
        return
    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.long_only:
        # (only the step as CustomAttention runs it, so that a kernel trace of this command holds one plan per kernel)
        print(json.dumps(long_context(torch, ct, dev, args.long_only, args.steps, args.warmup, compare_plain=False)))
        return
    B, H, N, D = 8, 16, 2048, 64
    q, k, v, do = make_inputs(torch, B, H, N, D, D, torch.bfloat16, dev)
    if args.cold_only:
        def fwd_saving():
            return ct.causal_dot_product_saving(q, k, v)
        saved = fwd_saving()[1]
        print(json.dumps({"cold_cache_headline": cold_cache_kernel_times(
            torch, fwd_saving, lambda: ct.causal_backward(q, k, v, do, saved=saved), dev, B * H * N * D * 2, 256)}))
        return

    # The step as CustomAttention runs it on 16-bit tensors: the forward pass leaves the state dQ starts from (here one
    # 16 KiB slot per head, the sum over the whole sequence) and the backward pass takes it, so that dQ walks the
    # sequence from the end together with dK and dV.  The plain entry points are timed beside it (extras).
    saving = ct.saved_states_plan(torch.bfloat16, B, H, N, D, D) is not None
    if saving:
        saved0 = ct.causal_dot_product_saving(q, k, v)[1]
        fwd = lambda: ct.causal_dot_product_saving(q, k, v)
        bwd = lambda: ct.causal_backward(q, k, v, do, saved=saved0)

        def step():
            o, saved = ct.causal_dot_product_saving(q, k, v)
            grads = ct.causal_backward(q, k, v, do, saved=saved)
            return o, grads
    else:
        fwd = lambda: ct.causal_dot_product(q, k, v)
        bwd = lambda: ct.causal_backward(q, k, v, do)

        def step():
            return fwd(), bwd()

    # untimed spin-up so that the clocks have settled before the W warm-up steps (a cold process measures ~8 % low)
    t_end = time.perf_counter() + SPINUP_S
    while time.perf_counter() < t_end:
        for _ in range(50):
            step()
        torch.cuda.synchronize()

    sec = time_region(torch, step, args.steps, args.warmup)
    tokens_per_s = B * N / sec

    # forward-only / backward-only split (same buffers)
    sec_f = time_region(torch, fwd, args.steps, 5)
    sec_b = time_region(torch, bwd, args.steps, 5)
    if saving:
        def plain_step():
            ct.causal_dot_product(q, k, v)
            ct.causal_backward(q, k, v, do)
        sec_plain = time_region(torch, plain_step, args.steps, args.warmup)
        sec_plain_b = time_region(torch, lambda: ct.causal_backward(q, k, v, do), args.steps, 5)

    # Per-kernel durations: the library brackets each launch with HIP events on the launch stream.
    _loader.profile_enable(True)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    _loader.profile_enable(False)
    kern = {}
    for name in _loader.KERNEL_IDS:
        ms, n = _loader.profile_read(name)
        if n:
            kern[name] = {"launches_per_step": n / args.steps, "avg_us": 1e3 * ms / n, "us_per_step": 1e3 * ms / args.steps}
    dominant = max(kern, key=lambda kname: kern[kname]["us_per_step"])
    esz = 2
    tensor_bytes = B * H * N * D * esz
    # algorithmic bytes of ONE launch of each kernel family at this shape (tensor passes x 32 MiB)
    # scan (forward launch): read Q,K,V + write O; scan_grad (one launch for dQ,dK,dV): read Q,K,V,dO + write 3
    passes = {"scan": 4, "scan_grad": 7, "group_state": 2}
    alg_bytes = passes.get(dominant, 4) * tensor_bytes
    achieved = alg_bytes / (kern[dominant]["avg_us"] * 1e-6) / 1e9
    # the same kernels with cold caches: what a training step sees (other kernels run between forward and backward)
    cold = cold_cache_kernel_times(torch, fwd, bwd, dev, tensor_bytes, 256)
    cold_dom = cold["bwd_kernel_us"] if dominant == "scan_grad" else cold["fwd_kernel_us"]
    cold_step_us = cold["fwd_kernel_us"] + cold["bwd_kernel_us"]
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES.get(dominant),
                "kernel": dominant, "avg_us": kern[dominant]["avg_us"],
                "algorithmic_bytes_per_launch": alg_bytes,
                "cold_avg_us": cold_dom, "cold_achieved": alg_bytes / (cold_dom * 1e-6) / 1e9,
                "cold_frac": alg_bytes / (cold_dom * 1e-6) / 1e9 / HBM_PEAK_GBS,
                "cold_whole_step": {"fwd_kernel_us": cold["fwd_kernel_us"], "bwd_kernel_us": cold["bwd_kernel_us"],
                                    "tokens_per_s": B * N / (cold_step_us * 1e-6),
                                    "frac_hbm": 11 * tensor_bytes / (cold_step_us * 1e-6) / 1e9 / HBM_PEAK_GBS},
                "whole_step": {"algorithmic_bytes": 11 * tensor_bytes,
                               "achieved_GBps": 11 * tensor_bytes / sec / 1e9,
                               "frac_hbm": 11 * tensor_bytes / sec / 1e9 / HBM_PEAK_GBS,
                               "algorithmic_tflops": 14.0 * B * H * N * D * D / sec / 1e12,
                               "frac_mfma_bf16": 14.0 * B * H * N * D * D / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS}}

    extras = {"fwd_us": sec_f * 1e6, "bwd_us": sec_b * 1e6, "kernels": kern, "states_saved_for_backward": saving}
    if saving:
        extras["plain_entry_points"] = {"us_per_step": sec_plain * 1e6, "bwd_us": sec_plain_b * 1e6,
                                        "tokens_per_s": B * N / sec_plain}
    extras["cold_cache_headline"] = cold
    if not args.no_extras:
        extras.update(run_extras(torch, ct, dev))

    out = {
        "metric": "causal cos-attn fwd+bwd tokens/s, B8 H16 N2048 D64 bf16; % MFMA/HBM peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[2]: GPT-300M-shape causal cosine attention fwd+bwd (dQ,dK,dV), "
                               "B=8 H=16 N=2048 D=64 bf16, fp32 state carry; forward keeps a 16 KiB state per head "
                               "for the backward pass, as CustomAttention does", "B": B, "H": H, "N": N, "D": D,
                   "spinup_s": SPINUP_S},
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(torch),
        "extras": extras,
    }
    print(json.dumps(out))


def cold_kernel_us(torch, fn, kernel, big):
    """Average duration of one kernel family when nothing is left in L2 or the 256 MB last-level cache from the
    previous call (a read of 1 GiB of other data, `big`, runs before every launch; a read, so that no dirty lines of
    the evicting kernel are written back during the measurement), which is how a training step meets these kernels.
    A loop over the same tensors is served partly from that cache."""
    from cottention_transformer_amd import _loader
    fn()
    torch.cuda.synchronize()
    _loader.profile_enable(True)
    for _ in range(20):
        big.sum()
        fn()
    torch.cuda.synchronize()
    _loader.profile_enable(False)
    ms, n = _loader.profile_read(kernel)
    return 1e3 * ms / n


def cold_cache_kernel_times(torch, fwd, bwd, dev, tensor_bytes, workgroups):
    """Forward and gradient launches with cold caches, and beside them a kernel of the same launch shape that only
    streams the same tensors (cott_stream_probe: `workgroups` workgroups, each walking its contiguous share of three /
    four tensors in 8 KiB blocks, two in flight, and writing one / three), measured the same way: the memory system's
    part of the cold durations."""
    from cottention_transformer_amd import _loader
    big = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
    out = {"fwd_kernel_us": cold_kernel_us(torch, fwd, "scan", big),
           "bwd_kernel_us": cold_kernel_us(torch, bwd, "scan_grad", big)}
    src = torch.ones(4 * tensor_bytes // 4, dtype=torch.int32, device=dev)
    dst = torch.zeros(3 * tensor_bytes // 4, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def probe(nr, nw):
        def fn():
            rc = _loader.lib().cott_stream_probe(src.data_ptr(), dst.data_ptr(), tensor_bytes, nr, nw, workgroups, 8192, stream)
            if rc != _loader.OK:
                raise RuntimeError("cott_stream_probe refused the launch")
        return fn
    out["streaming_only"] = {
        "workgroups": workgroups, "block_bytes": 8192,
        "fwd_shape_3_reads_1_write_us": cold_kernel_us(torch, probe(3, 1), "stream_probe", big),
        "grad_shape_4_reads_3_writes_us": cold_kernel_us(torch, probe(4, 3), "stream_probe", big)}
    out["fwd_over_streaming_only"] = out["fwd_kernel_us"] / out["streaming_only"]["fwd_shape_3_reads_1_write_us"]
    out["bwd_over_streaming_only"] = out["bwd_kernel_us"] / out["streaming_only"]["grad_shape_4_reads_3_writes_us"]
    del big, src, dst
    return out


def long_context(torch, ct, dev, n, steps, warmup, kernels=True, compare_plain=True):
    """Long-context configuration B=1 H=16 D=128 bf16 at sequence length n: forward, backward and both, with the
    per-kernel durations the library records (HIP events around each launch)."""
    from cottention_transformer_amd import _loader
    q, k, v, do = make_inputs(torch, 1, 16, n, 128, 128, torch.bfloat16, dev)
    tb = 16 * n * 128 * 2

    def measure(fwd, bwd):
        def both():
            fwd()
            bwd()
        t_end = time.perf_counter() + SPINUP_S  # untimed spin-up, as for the headline: clocks settle
        while time.perf_counter() < t_end:
            both()
            torch.cuda.synchronize()
        s = time_region(torch, both, steps, warmup)
        return {"us": s * 1e6, "fwd_us": time_region(torch, fwd, steps, 2) * 1e6,
                "bwd_us": time_region(torch, bwd, steps, 2) * 1e6, "tokens_per_s": n / s, "GBps": 11 * tb / s / 1e9,
                "frac_hbm": 11 * tb / s / 1e9 / HBM_PEAK_GBS}
    # The step as CustomAttention runs it: where the backward pass is cut into sequence groups, the forward pass
    # leaves the states at the cuts (a few MiB) and the backward pass starts dQ from them.
    saving = ct.saved_states_plan(torch.bfloat16, 1, 16, n, 128, 128) is not None
    if saving:
        saved = ct.causal_dot_product_saving(q, k, v)[1]
        fwd = lambda: ct.causal_dot_product_saving(q, k, v)
        bwd = lambda: ct.causal_backward(q, k, v, do, saved=saved)
    else:
        fwd = lambda: ct.causal_dot_product(q, k, v)
        bwd = lambda: ct.causal_backward(q, k, v, do)
    out = {"N": n, "states_saved_for_backward": saving}
    out.update(measure(fwd, bwd))
    if saving and compare_plain:
        plain = measure(lambda: ct.causal_dot_product(q, k, v), lambda: ct.causal_backward(q, k, v, do))
        out["plain_entry_points"] = {k_: plain[k_] for k_ in ("us", "fwd_us", "bwd_us", "frac_hbm")}
    if kernels:
        for name, fn in (("fwd_kernels_us", fwd), ("bwd_kernels_us", bwd)):
            _loader.profile_enable(True)
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            _loader.profile_enable(False)
            out[name] = {}
            for kname in _loader.KERNEL_IDS:
                ms, cnt = _loader.profile_read(kname)
                if cnt:
                    out[name][kname] = 1e3 * ms / steps
    return out


def gpt_block_step(torch, dev):
    """step(use_cache): forward + backward of one GPT attention block (B8 S2048 E1024 H16) under bf16 autocast.
    use_cache=True makes the module return the rotated keys, i.e. rotary and head permutes run as torch ops."""
    from types import SimpleNamespace
    from cottention_transformer_amd import modules
    cfg = SimpleNamespace(max_position_embeddings=2048, attn_pdrop=0.0, resid_pdrop=0.0, hidden_size=1024,
                          num_attention_heads=16, rotary_dim=64)
    blk = modules.GPTCosAttention(cfg).to(dev)
    hid = torch.randn(8, 2048, 1024, device=dev, requires_grad=True)
    gout = torch.randn(8, 2048, 1024, device=dev, dtype=torch.bfloat16)
    # the ids as GPT-J's model hands them to every block: one arange row for the whole batch (GPTCosAttention.py:458)
    position_ids = torch.arange(0, 2048, dtype=torch.long, device=dev).unsqueeze(0)

    def step(use_cache):
        # gradients start from None, as after a training loop's zero_grad(set_to_none=True): the hidden states of a
        # model are no leaf, so accumulating into hid.grad would add a 64 MiB pass that no training step has
        hid.grad = None
        blk.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = blk(hid, position_ids=position_ids, use_cache=use_cache)[0]
        out.backward(gout)
    return step


def bert_block_step(torch, dev):
    """step(): forward + backward of the BERT self-attention block (projections, preparation, non-causal attention)
    under bf16 autocast at the BERT-base shape B32 S512 E768 H12, with the padding mask of a batch whose sequences
    end between half and full length."""
    from types import SimpleNamespace
    from cottention_transformer_amd import modules
    bert = modules.BertCosAttention(SimpleNamespace(hidden_size=768, num_attention_heads=12,
                                                    attention_probs_dropout_prob=0.0)).to(dev)
    hid = torch.randn(32, 512, 768, device=dev, requires_grad=True)
    gout = torch.randn(32, 512, 768, device=dev, dtype=torch.bfloat16)
    keep = torch.arange(512, device=dev)[None, :] < torch.randint(256, 513, (32, 1), device=dev)
    mask = ((~keep).float() * torch.finfo(torch.float32).min)[:, None, None, :]

    def step():
        hid.grad = None
        bert.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = bert(hid, attention_mask=mask)[0]
        out.backward(gout)
    return step


def module_anchor(torch, dev):
    """Forward latency of the two attention modules at batch 1, hidden 2048, 16 heads (D = 128), the one point the
    reference publishes for this path: its module-level plots (tests/MemoryTest.py:118-143, 233-278: eval mode, fp32,
    no autocast, time.time() without device synchronisation, GPU not stated) read about 13 ms (Cos-GPT) and 11 ms
    (Cos-BERT) at S = 16384.  Here: synchronised, median of 10 after 3 warm-ups, fp32 as there and under bf16
    autocast."""
    from types import SimpleNamespace
    from cottention_transformer_amd import modules
    gpt = modules.GPTCosAttention(SimpleNamespace(max_position_embeddings=16384, attn_pdrop=0.0, resid_pdrop=0.0,
                                                  hidden_size=2048, num_attention_heads=16, rotary_dim=64)).to(dev).eval()
    bert = modules.BertCosAttention(SimpleNamespace(hidden_size=2048, num_attention_heads=16,
                                                    attention_probs_dropout_prob=0.0)).to(dev).eval()
    out = {"reference_plot_readoff_ms_at_S16384": {"cos_gpt": 13.0, "cos_bert": 11.0, "hardware": "unstated GPU"}}

    def lat(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(10):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        return statistics.median(ts) * 1e3

    with torch.no_grad():
        for s_len in (1024, 2048, 4096, 8192, 16384):
            x = torch.randn(1, s_len, 2048, device=dev)
            row = {"cos_gpt_fp32_ms": lat(lambda: gpt(x)), "cos_bert_fp32_ms": lat(lambda: bert(x))}
            with torch.autocast("cuda", dtype=torch.bfloat16):
                row["cos_gpt_bf16_autocast_ms"] = lat(lambda: gpt(x))
                row["cos_bert_bf16_autocast_ms"] = lat(lambda: bert(x))
            out[f"S{s_len}"] = row
            del x
    return out


def run_extras(torch, ct, dev):
    """Secondary configurations of the same path (not the headline value)."""
    ex = {}
    # non-causal forward, B=32 H=12 N=512 D=64 bf16
    b, h, n, d = 32, 12, 512, 64
    q, k, v = make_inputs(torch, b, h, n, d, d, torch.bfloat16, dev, grad=False)
    s = time_region(torch, lambda: ct.noncausal_dot_product(q, k, v), 100, 10)
    byts = 4 * b * h * n * d * 2
    ex["noncausal_fwd_B32_H12_N512_D64"] = {"us": s * 1e6, "tokens_per_s": b * n / s, "GBps": byts / s / 1e9,
                                            "frac_hbm": byts / s / 1e9 / HBM_PEAK_GBS}
    do = torch.randn_like(v)
    s = time_region(torch, lambda: ct.noncausal_backward(q, k, v, do), 100, 10)
    byts = 7 * b * h * n * d * 2
    ex["noncausal_bwd_B32_H12_N512_D64"] = {"us": s * 1e6, "tokens_per_s": b * n / s, "GBps": byts / s / 1e9,
                                            "frac_hbm": byts / s / 1e9 / HBM_PEAK_GBS}
    big = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
    cf = cold_kernel_us(torch, lambda: ct.noncausal_dot_product(q, k, v), "apply", big)
    cb = cold_kernel_us(torch, lambda: ct.noncausal_backward(q, k, v, do), "apply", big)
    tb = b * h * n * d * 2
    # beside them the kernel that only streams the same tensors in a launch of as many workgroups as there are heads
    # (cott_stream_probe; the non-causal kernels read k, v and then q in two passes, the probe in one)
    from cottention_transformer_amd import _loader
    src = torch.ones(4 * tb // 4, dtype=torch.int32, device=dev)
    dst = torch.zeros(3 * tb // 4, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def probe(nr, nw):
        def fn():
            if _loader.lib().cott_stream_probe(src.data_ptr(), dst.data_ptr(), tb, nr, nw, b * h, 8192, stream) != _loader.OK:
                raise RuntimeError("cott_stream_probe refused the launch")
        return fn
    ex["noncausal_cold_cache_B32_H12_N512_D64"] = {
        "fwd_kernel_us": cf, "fwd_frac_hbm": 4 * tb / (cf * 1e-6) / 1e9 / HBM_PEAK_GBS, "fwd_tokens_per_s": b * n / (cf * 1e-6),
        "bwd_kernel_us": cb, "bwd_frac_hbm": 7 * tb / (cb * 1e-6) / 1e9 / HBM_PEAK_GBS,
        "streaming_only": {"workgroups": b * h, "block_bytes": 8192,
                           "fwd_shape_3_reads_1_write_us": cold_kernel_us(torch, probe(3, 1), "stream_probe", big),
                           "grad_shape_4_reads_3_writes_us": cold_kernel_us(torch, probe(4, 3), "stream_probe", big)}}
    del q, k, v, do, big, src, dst
    # recurrent decode, state (256,16,128,128) fp32, 512 consecutive steps with fresh q,k,v per step
    b, h, d, steps = 256, 16, 128, 512
    g = torch.Generator(device=dev).manual_seed(0)
    S = (0.01 * torch.randn(b, h, d, d, generator=g, device=dev, dtype=torch.float32)).contiguous()
    qs = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g, device=dev), dim=-1).to(torch.bfloat16)
    ks = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g, device=dev), dim=-1).to(torch.bfloat16)
    vs = torch.randn(steps, b, h, d, generator=g, device=dev).to(torch.bfloat16)
    out = torch.empty(b, h, d, dtype=torch.bfloat16, device=dev)
    for t in range(8):
        ct.decode_step(S, qs[t], ks[t], vs[t], out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(steps):
        ct.decode_step(S, qs[t], ks[t], vs[t], out=out)
    torch.cuda.synchronize()
    s = time.perf_counter() - t0
    byts = steps * (2 * b * h * d * d * 4 + 4 * b * h * d * 2)
    ex["decode_B256_H16_D128_512steps"] = {"ms_total": s * 1e3, "us_per_step": s / steps * 1e6,
                                           "tokens_per_s": b * steps / s, "GBps": byts / s / 1e9,
                                           "frac_hbm": byts / s / 1e9 / HBM_PEAK_GBS,
                                           "note": "state is 256 MiB = the size of the last-level cache; "
                                                   "GB/s is algorithmic bytes / time"}
    del S, qs, ks, vs
    # the same step on a state four times the last-level cache (B=1024: 1 GiB), where every byte comes from memory
    b, steps = 1024, 64
    S = (0.01 * torch.randn(b, h, d, d, generator=g, device=dev, dtype=torch.float32)).contiguous()
    qs = torch.nn.functional.normalize(torch.randn(8, b, h, d, generator=g, device=dev), dim=-1).to(torch.bfloat16)
    ks = torch.nn.functional.normalize(torch.randn(8, b, h, d, generator=g, device=dev), dim=-1).to(torch.bfloat16)
    vs = torch.randn(8, b, h, d, generator=g, device=dev).to(torch.bfloat16)
    out = torch.empty(b, h, d, dtype=torch.bfloat16, device=dev)
    for t in range(4):
        ct.decode_step(S, qs[t], ks[t], vs[t], out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(steps):
        ct.decode_step(S, qs[t % 8], ks[t % 8], vs[t % 8], out=out)
    torch.cuda.synchronize()
    s = time.perf_counter() - t0
    byts = steps * (2 * b * h * d * d * 4 + 4 * b * h * d * 2)
    ex["decode_B1024_H16_D128_state_1GiB"] = {"us_per_step": s / steps * 1e6, "tokens_per_s": b * steps / s,
                                              "GBps": byts / s / 1e9, "frac_hbm": byts / s / 1e9 / HBM_PEAK_GBS,
                                              "note": "state is 4x the last-level cache: achieved HBM rate"}
    del S, qs, ks, vs, out
    # long context fwd+bwd, B=1 H=16 D=128 bf16, N sweep
    sweep = {}
    for n in (4096, 8192, 16384, 32768, 65536):
        sweep[str(n)] = long_context(torch, ct, dev, n, 20, 3, kernels=(n == 65536))
    rates = [x["tokens_per_s"] for x in sweep.values()]
    sweep["tokens_per_s_min_over_max"] = min(rates) / max(rates)
    ex["long_context_fwd_bwd_B1_H16_D128"] = sweep
    # fp32 storage at the headline shape (what the backward of an autocast training step runs: the autograd
    # function saves the fp32 inputs, Cuda_Kernel/Custom_Kernel.py:16,38); fp32 MFMA, peak 157.3 TFLOP/s
    q, k, v, do = make_inputs(torch, 8, 16, 2048, 64, 64, torch.float32, dev)

    def step32():
        ct.causal_dot_product(q, k, v)
        ct.causal_backward(q, k, v, do)
    s = time_region(torch, step32, 20, 3)
    byts = 11 * 8 * 16 * 2048 * 64 * 4
    flops = 28.0 * 8 * 16 * 2048 * 64 * 64   # executed by the chunked form (scores recomputed per gradient)
    # fused input preparation (normalise q,k; scale v; mask; fp32 -> bf16) at the headline shape, next to the same
    # sequence written with torch elementwise ops as the reference module does (GPTCosAttention.py:229-248)
    keep = torch.rand(8, 2048, device=dev) > 0.1
    cnt = keep.float().cumsum(-1)
    sig = torch.sigmoid(torch.randn(16, device=dev))
    s_f = time_region(torch, lambda: ct.prepare_inputs(q, k, v, keep, cnt, sig, out_dtype=torch.bfloat16), 50, 5)

    def eager_prep():
        m = keep[:, None, :, None]
        qh = torch.nn.functional.normalize(q, dim=-1, p=2) * m
        kh = torch.nn.functional.normalize(k, dim=-1, p=2) * m
        vs = v / (cnt[:, None, :, None] ** sig.reshape(1, -1, 1, 1)).clamp(min=1) * m
        return qh.bfloat16(), kh.bfloat16(), vs.bfloat16()
    s_e = time_region(torch, eager_prep, 20, 3)
    pb = 3 * 8 * 16 * 2048 * 64 * (4 + 2)
    ex["input_prep_fwd_B8_H16_N2048_D64_f32_to_bf16"] = {"us": s_f * 1e6, "GBps": pb / s_f / 1e9,
                                                         "frac_hbm": pb / s_f / 1e9 / HBM_PEAK_GBS,
                                                         "torch_elementwise_us": s_e * 1e6}
    del keep, cnt, sig
    # the BERT block's preparation inside the non-causal kernel (cott_noncausal_fwd_prep) at the BERT-base shape, on
    # the projections' (B,S,H,D) tensors with a padding mask, next to the separate pass followed by the plain kernel
    bq, bk, bv = (torch.randn(32, 512, 12, 64, device=dev).bfloat16() for _ in range(3))
    bkeep = torch.arange(512, device=dev)[None, :] < torch.randint(256, 513, (32, 1), device=dev)
    bcnt = bkeep.sum(-1, keepdim=True).float().expand(32, 512).contiguous()
    bsig = torch.sigmoid(torch.randn(12, device=dev))

    def nc_two_kernels():
        p = ct.prepare_inputs(bq, bk, bv, bkeep, bcnt, bsig, out_dtype=torch.bfloat16, bnhd=True)
        return ct.noncausal_dot_product(*p, merged_heads=True)
    s_nf = time_region(torch, lambda: ct.noncausal_dot_product_prepared(bq, bk, bv, bkeep, bcnt, bsig, bnhd=True,
                                                                        merged_heads=True), 100, 10)
    s_n2 = time_region(torch, nc_two_kernels, 100, 10)
    ex["noncausal_fwd_with_preparation_B32_H12_N512_D64"] = {"one_launch_us": s_nf * 1e6,
                                                             "separate_pass_plus_kernel_us": s_n2 * 1e6}
    del bq, bk, bv, bkeep, bcnt, bsig
    # the GPT block's preparation (rotary with position ids, normalisation, value scaling, mask) inside the causal
    # forward (cott_causal_fwd_prep) on the projections' (B,S,H,D) tensors, next to the separate pass followed by the
    # plain forward: the headline shape and the GPT-1.2B head shape at the long-context length
    for (cb, ch, cn, cd) in ((8, 16, 2048, 64), (1, 16, 65536, 128)):
        cq, ck, cv = (torch.randn(cb, cn, ch, cd, device=dev).bfloat16() for _ in range(3))
        ckeep = torch.rand(cb, cn, device=dev) > 0.1
        ccnt = ckeep.float().cumsum(-1).contiguous()
        csig = torch.sigmoid(torch.randn(ch, device=dev))
        ctab = torch.randn(cn, 32, device=dev)
        cpos = torch.arange(cn, device=dev).expand(cb, cn).contiguous()

        def c_two_kernels():
            p = ct.prepare_inputs(cq, ck, cv, ckeep, ccnt, csig, rotary=(ctab, cpos), bnhd=True, check_positions=False)
            return ct.causal_dot_product(*p, merged_heads=True)
        s_cf = time_region(torch, lambda: ct.causal_dot_product_prepared(cq, ck, cv, ckeep, ccnt, csig, rotary=(ctab, cpos),
                                                                         bnhd=True, merged_heads=True), 30, 5)
        s_c2 = time_region(torch, c_two_kernels, 30, 5)
        ex[f"causal_fwd_with_preparation_B{cb}_H{ch}_N{cn}_D{cd}"] = {
            "one_launch_us": s_cf * 1e6, "separate_pass_plus_kernel_us": s_c2 * 1e6,
            "modules_take_the_one_launch": bool(ct.fused_preparation_preferred(torch.bfloat16, cb, ch, cn, cd, cd, 32))}
        del cq, ck, cv, ckeep, ccnt, csig, ctab, cpos
    # whole GPT attention block (projections, rotary, preparation, attention, output projection), fwd+bwd under
    # bf16 autocast at the GPT-300M shape; second figure: same block with rotary / head permute as torch ops
    block_step = gpt_block_step(torch, dev)
    s_fused = time_region(torch, lambda: block_step(False), 20, 3)
    s_torch = time_region(torch, lambda: block_step(True), 20, 3)
    ex["gpt_block_fwd_bwd_B8_S2048_E1024_H16_autocast_bf16"] = {
        "us": s_fused * 1e6, "tokens_per_s": 8 * 2048 / s_fused,
        "us_with_rotary_and_permute_as_torch_ops": s_torch * 1e6}
    del block_step
    bert_step = bert_block_step(torch, dev)
    s_b = time_region(torch, bert_step, 20, 3)
    ex["bert_block_fwd_bwd_B32_S512_E768_H12_autocast_bf16"] = {"us": s_b * 1e6, "tokens_per_s": 32 * 512 / s_b}
    del bert_step
    ex["module_forward_latency_batch1_hidden2048_heads16"] = module_anchor(torch, dev)
    # prompt pass that also hands the state to decoding (cott_causal_fwd_state), headline shape
    qp, kp, vp, _ = make_inputs(torch, 8, 16, 2048, 64, 64, torch.bfloat16, dev)
    s_p = time_region(torch, lambda: ct.causal_prefill(qp, kp, vp), 100, 10)
    ex["prefill_with_state_B8_H16_N2048_D64"] = {"us": s_p * 1e6, "tokens_per_s": 8 * 2048 / s_p}
    del qp, kp, vp
    ex["fp32_fwd_bwd_B8_H16_N2048_D64"] = {"us": s * 1e6, "tokens_per_s": 8 * 2048 / s, "GBps": byts / s / 1e9,
                                           "frac_hbm": byts / s / 1e9 / HBM_PEAK_GBS,
                                           "executed_tflops": flops / s / 1e12,
                                           "frac_mfma_fp32": flops / s / 1e12 / 157.3}
    del q, k, v, do
    # For scale: what plain torch kernels stream on this GPU over 1 GiB buffers (far beyond the caches)
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    gb = src.numel() * 4 / 1e9
    ex["torch_streaming_1GiB_GBps"] = {
        "read_sum": gb / time_region(torch, lambda: src.sum(), 10, 2),
        "write_fill": gb / time_region(torch, lambda: dst.fill_(1.0), 10, 2),
        "copy_read_plus_write": 2 * gb / time_region(torch, lambda: dst.copy_(src), 10, 2)}
    del src, dst
    return ex


if __name__ == "__main__":
    main()
