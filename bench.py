"""Benchmark of the stick-breaking attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg4|cfg5|short|d256] [--dtype bf16|f16]

A step is one forward + backward of the operator through its public autograd API on
synthetic inputs already resident in HBM.  Prints ONE JSON line.
"""
import argparse
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

BF16_MFMA_PEAK_TFLOPS = 2516.6     # 256 CU x 2.4 GHz x 4096 FLOP/clk/CU (dense bf16)
HBM_PEAK_GBS = 8000.0               # MI355X HBM3E

KERNEL_TIMING_SAMPLES = 5      # steps of the timed region whose kernels are timed with events
# Counters cannot be read from inside this process: HBM bytes and instruction counts per launch are read from the
# rocprofv3 summaries kept under profiles/ (sba_<workload>_hbm_traffic.txt, sba_<workload>_shader_counters.txt) and
# are reported with that source next to what this run measures itself; a missing or unreadable file gives null.
PROFILE_DIR = os.path.join(ROOT, "profiles")
KERNEL_COLUMN = {"fwd": "fwd", "bwd_dq": "dq", "bwd_dkv": "dkv"}


def profiled_hbm_bytes(workload, kernel):
    """FETCH_SIZE + WRITE_SIZE per launch, scaled by a copy kernel of known size: the line
    'traffic per launch (read+write) in bytes: fwd N, bwd_dq N, bwd_dkv N' of the summary."""
    try:
        text = open(os.path.join(PROFILE_DIR, f"sba_{workload}_hbm_traffic.txt")).read()
    except OSError:
        return None
    m = re.search(r"traffic per launch \(read\+write\) in bytes:([^\n(]*)", text)
    if not m:
        return None
    found = dict(re.findall(r"(\w+) (\d+)", m.group(1)))
    return int(found[kernel]) if kernel in found else None


def profiled_instructions(workload, kernel):
    """Wave instructions per launch (vector incl. transcendental, transcendental, MFMA) from the counter table of
    the summary (rows SQ_INSTS_VALU, SQ_INSTS_VALU_TRANS_F32, SQ_INSTS_MFMA; columns dkv, dq, fwd)."""
    try:
        lines = open(os.path.join(PROFILE_DIR, f"sba_{workload}_shader_counters.txt")).read().splitlines()
    except OSError:
        return None
    cols, rows = None, {}
    for ln in lines:
        f = ln.split()
        if f and f[0] == "counter":
            cols = f[1:]
        elif cols and len(f) == len(cols) + 1 and f[0].startswith("SQ_"):
            rows[f[0]] = dict(zip(cols, f[1:]))
    try:
        c = KERNEL_COLUMN[kernel]
        return tuple(int(float(rows[r][c])) for r in ("SQ_INSTS_VALU", "SQ_INSTS_VALU_TRANS_F32", "SQ_INSTS_MFMA"))
    except (KeyError, ValueError):
        return None


# Issue time of one SIMD per instruction in cycles, four waves per SIMD (profiles/gfx950_issue_rates.txt): plain
# vector, transcendental issued while MFMAs are in flight, MFMA 32x32x16 bf16; the chip holds about 2.0 GHz under
# this mix.  MFMAs and plain vector instructions do not overlap on gfx950, also across waves: their times add up.
ISSUE_CYCLES = {"vector": 2.3, "transcendental": 2.2, "mfma": 34.0}
MIXED_CLOCK_GHZ = 2.0
N_SIMDS = 1024
# The fewest vector instructions per (query, key) pair the algorithm needs in each kernel (of them transcendental):
# forward exp, two fma, a multiply and half a pack; each backward pass exp, rcp, six arithmetic instructions and a pack.
MINIMUM_PER_PAIR = {"fwd": (4.5, 1.0), "bwd_dq": (10.5, 2.0), "bwd_dkv": (10.0, 2.0)}


def issue_ms(valu, trans, mfma):
    cycles = (valu - trans) * ISSUE_CYCLES["vector"] + trans * ISSUE_CYCLES["transcendental"] + mfma * ISSUE_CYCLES["mfma"]
    return cycles / N_SIMDS / (MIXED_CLOCK_GHZ * 1e9) * 1e3


def issue_floors(workload, kernel, pairs):
    """Secondary ceilings: the time the kernel's instructions need at the measured issue rates, for the counts it
    executes today and for the algorithm's minimum vector counts (same MFMAs)."""
    c = profiled_instructions(workload, kernel)
    if c is None:
        return None
    valu, trans, mfma = c
    per_pair, trans_per_pair = MINIMUM_PER_PAIR[kernel]
    return {"present_counts": issue_ms(valu, trans, mfma),
            "minimum_counts": issue_ms(per_pair * pairs / 64, trans_per_pair * pairs / 64, mfma)}


def _lognormal_lengths(total, seed, median=600.0, sigma=1.0, lo=16, hi=4096):
    import torch
    g = torch.Generator().manual_seed(seed)
    lens, s = [], 0
    while s < total:
        L = int(round(math.exp(math.log(median) + sigma * torch.randn((), generator=g).item())))
        L = max(lo, min(hi, L))
        L = min(L, total - s)
        if L < lo and lens:
            lens[-1] += L       # a truncated tail shorter than `lo` joins the previous document
        else:
            lens.append(L)
        s += L
    return lens


def make_workload(name, device, dtype_name="bf16"):
    """Returns (description, step_fn inputs, number of allowed pairs P, tokens, d)."""
    import torch
    g = torch.Generator().manual_seed(0)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16}[dtype_name]

    def rn(shape, scale):
        return (torch.randn(shape, generator=g) * scale).to(dtype).to(device)

    if name == "d256":
        # head_dim 256 (no configuration of BASELINE.json; the size the reference would run with BLOCK_D = 256)
        B, H, T, D = 1, 8, 8192, 256
        q, k, v = rn((B, H, T, D), 0.5), rn((B, H, T, D), 0.5), rn((B, H, T, D), 0.5)
        do = rn((B, H, T, D), 1.0)
        pairs = B * H * T * (T - 1) // 2
        desc = {"workload": f"d256: dense causal fwd+bwd B=1 H=8 T=8192 d=256 {dtype_name}", "B": B, "H": H, "T": T, "d": D}
        return desc, (q, k, v, do, None, None), pairs, B * T, D, H

    if name == "cfg2":
        B, H, T, D = 1, 16, 4096, 64
        q, k, v = rn((B, H, T, D), 0.5), rn((B, H, T, D), 0.5), rn((B, H, T, D), 0.5)
        do = rn((B, H, T, D), 1.0)
        pairs = B * H * T * (T - 1) // 2
        desc = {"workload": f"cfg2: dense causal fwd+bwd B=1 H=16 T=4096 d=64 {dtype_name}", "B": B, "H": H, "T": T, "d": D}
        return desc, (q, k, v, do, None, None), pairs, B * T, D, H
    if name == "cfg4":
        B, H, T, D = 1, 16, 16384, 128
        q, k, v = rn((B, H, T, D), 0.5), rn((B, H, T, D), 0.5), rn((B, H, T, D), 1.0)
        # 1% of the key rows of every head get 3*u added, u a seeded unit vector per head
        n_sel = T // 100
        for h in range(H):
            sel = torch.randperm(T, generator=g)[:n_sel].to(device)
            u = torch.randn(D, generator=g)
            u = (3.0 * u / u.norm()).to(dtype).to(device)
            k[0, h, sel] += u
        do = rn((B, H, T, D), 1.0)
        pairs = B * H * T * (T - 1) // 2
        desc = {"workload": f"cfg4: dense causal fwd+bwd B=1 H=16 T=16384 d=128 {dtype_name}, 1% boosted keys",
                "B": B, "H": H, "T": T, "d": D}
        return desc, (q, k, v, do, None, None), pairs, B * T, D, H
    if name == "cfg3":
        H, N, D = 16, 65536, 64
        lens = _lognormal_lengths(N, seed=0)
        cu = [0]
        for L in lens:
            cu.append(cu[-1] + L)
        q, k, v = rn((H, N, D), 0.5), rn((H, N, D), 0.5), rn((H, N, D), 0.5)
        do = rn((H, N, D), 1.0)
        pairs = H * sum(L * (L - 1) // 2 for L in lens)
        cu_t = torch.tensor(cu, dtype=torch.int32, device=device)
        desc = {"workload": f"cfg3: packed varlen fwd+bwd H=16 d=64 {dtype_name}, 65536 tokens, lognormal docs",
                "H": H, "tokens": N, "d": D, "n_docs": len(lens), "max_len": max(lens)}
        return desc, (q, k, v, do, cu_t, max(lens)), pairs, N, D, H
    if name == "short":
        # the short-document regime of a packed batch: too few pairs per token for the matrix cores to
        # matter, every tensor is read once -> priced against the HBM roofline
        H, N, D = 16, 65536, 64
        lens, s_ = [], 0
        while s_ < N:
            L = min(int(torch.randint(16, 129, (1,), generator=g)), N - s_)
            lens.append(L)
            s_ += L
        cu = [0]
        for L in lens:
            cu.append(cu[-1] + L)
        q, k, v = rn((H, N, D), 0.5), rn((H, N, D), 0.5), rn((H, N, D), 0.5)
        do = rn((H, N, D), 1.0)
        pairs = H * sum(L * (L - 1) // 2 for L in lens)
        cu_t = torch.tensor(cu, dtype=torch.int32, device=device)
        desc = {"workload": f"short: packed varlen fwd+bwd H=16 d=64 {dtype_name}, 65536 tokens in documents of 16..128 tokens",
                "H": H, "tokens": N, "d": D, "n_docs": len(lens), "max_len": max(lens)}
        return desc, (q, k, v, do, cu_t, max(lens)), pairs, N, D, H
    raise SystemExit(f"unknown workload {name}")


def cpu_baseline(name, reps=3):
    """The oracle (a PyTorch restatement of the reference formula, oracle/sb_oracle.py) timed on
    the host cores on a bounded sample of workload `name`, scaled to the metric's unit through
    the same 12*d*P FLOP count.  cfg2: every head, full size.  cfg3: one head of the same packed
    batch (all documents).  cfg4: one head of a 4096-token prefix at d=128 (the full 16384-token
    head needs a 1 GiB score matrix per temporary)."""
    import torch
    from oracle import sb_oracle as O
    # the GPU box gives one GPU's job 16 cores, whatever os.cpu_count() shows there
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    g = torch.Generator().manual_seed(1)

    def rn(shape, scale=0.5):
        return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16)

    if name == "cfg3":
        D, N = 64, 65536
        lens = _lognormal_lengths(N, seed=0)
        cu = [0]
        for L in lens:
            cu.append(cu[-1] + L)
        q, k, v, do = rn((1, N, D)), rn((1, N, D)), rn((1, N, D)), rn((1, N, D), 1.0)
        run = lambda: O.sb_attn_grads_oracle(q, k, v, do, None, cu_seqlens=cu)
        pairs, full_pairs, tokens = sum(L * (L - 1) // 2 for L in lens), 16 * sum(L * (L - 1) // 2 for L in lens), N
        what = f"1 of 16 heads of the cfg3 pack ({len(lens)} documents, 65536 tokens, d=64), document by document"
    elif name == "cfg4":
        T, D, Hs = 4096, 128, 8
        q, k, v, do = rn((1, Hs, T, D)), rn((1, Hs, T, D)), rn((1, Hs, T, D), 1.0), rn((1, Hs, T, D), 1.0)

        def run():
            for h in range(Hs):
                O.sb_attn_grads_oracle(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], do[:, h:h + 1])
        pairs, full_pairs, tokens = Hs * T * (T - 1) // 2, 16 * 16384 * 16383 // 2, 16384
        what = "8 heads of a 4096-token prefix at d=128 (1/32 of cfg4's pairs: T=16384 needs 1 GiB per score matrix)"
    else:
        T, D, H = 4096, 64, 16
        q, k, v, do = rn((1, H, T, D)), rn((1, H, T, D)), rn((1, H, T, D)), rn((1, H, T, D), 1.0)

        def run():
            for h in range(H):
                O.sb_attn_grads_oracle(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], do[:, h:h + 1])
        pairs, full_pairs, tokens = H * T * (T - 1) // 2, H * T * (T - 1) // 2, T
        what = "all 16 heads of cfg2 (T=4096, d=64), one head at a time"
    D = q.shape[-1]
    O.sb_attn_grads_oracle(rn((1, 1, 256, D)), rn((1, 1, 256, D)), rn((1, 1, 256, D)), rn((1, 1, 256, D)))   # warm-up
    t0 = time.perf_counter()
    for _ in range(reps):
        run()
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(12 * D * pairs / dt / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "workload": name,
            "sample": f"oracle/sb_oracle.py (torch fp32) fwd+bwd of {what}, {reps} repetitions, {dt:.2f} s each; "
                      f"same 12*d*P FLOP count",
            "tokens_per_s": round(tokens / (dt * full_pairs / pairs), 1)}


def parity_sample(name, q, k, v, do, cu, o, rem):
    """One head of the TIMED tensors against the oracle (the checker of the test-suite, here on a sample small
    enough for a few seconds of CPU): cfg2 head 0 whole, forward and all gradients; cfg3 head 0, the first
    documents of the pack (up to 4096 tokens), forward and all gradients; cfg4 head 0, the first 2048 tokens -
    causality makes o, rem and dq of a prefix depend on the prefix alone (dk, dv do not: not compared there).
    Tolerances as in the tests: o / rem max-abs 2e-2, gradients 5e-2 relative L2."""
    import torch
    from oracle import sb_oracle as O
    f = lambda t: t.detach().float().cpu()
    rel = lambda a, b: float((a - b).norm() / b.norm().clamp_min(1e-30))
    if name == "cfg3":
        ends = [int(e) for e in cu.cpu().tolist()]
        n_docs = max(1, sum(1 for e in ends[1:] if e <= 4096))
        N = ends[n_docs]
        cut = lambda t: f(t[0:1, :N])
        ref = O.sb_attn_grads_oracle(cut(q), cut(k), cut(v), cut(do), None, cu_seqlens=ends[:n_docs + 1])
        got = (cut(o), f(rem[0:1, :N]), cut(q.grad), cut(k.grad), cut(v.grad))
        what, full = f"head 0, first {n_docs} documents ({N} tokens) of the timed pack", True
    else:
        P = 2048 if name == "cfg4" else q.shape[2]
        cut = lambda t: f(t[:, 0:1, :P])
        ref = O.sb_attn_grads_oracle(cut(q), cut(k), cut(v), cut(do))
        got = (cut(o), f(rem[:, 0:1, :P]), cut(q.grad), cut(k.grad), cut(v.grad))
        full = name != "cfg4"
        what = f"head 0 of the timed tensors, {'all' if full else 'the first'} {P} tokens" + ("" if full else " (o, rem, dq)")
    res = {"what": what, "o_max_abs": float((got[0] - ref[0]).abs().max()), "rem_max_abs": float((got[1] - ref[1]).abs().max()),
           "dq_rel_l2": rel(got[2], ref[2])}
    if full:
        res["dk_rel_l2"], res["dv_rel_l2"] = rel(got[3], ref[3]), rel(got[4], ref[4])
    res["within_tolerance"] = bool(res["o_max_abs"] <= 2e-2 and res["rem_max_abs"] <= 2e-2 and
                                   all(res[g] <= 5e-2 for g in res if g.endswith("rel_l2")))
    return {k_: (round(v_, 6) if isinstance(v_, float) else v_) for k_, v_ in res.items()}


def settle_clocks(step, seconds=0.3):
    """Untimed work in front of the warm-up steps: an idle GPU needs some tens of milliseconds of
    load before it runs at its sustained clocks, and ten warm-up steps of a 0.3 ms workload are
    over before that (measured: 0.300 ms per step right after start, 0.275 ms once settled)."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            step()
        torch.cuda.synchronize()


def bench_model(args, dev):
    """benchmark configuration 5: full SBA-340M training step, one packed row of 8192 tokens."""
    import torch
    from flame_amd.modeling_sba import SBAConfig, SBAForCausalLM
    from flame_amd.train_step import make_optimizer, train_step
    torch.manual_seed(0)
    cfg = SBAConfig()
    model = SBAForCausalLM(cfg).to(dev)
    opt = make_optimizer(model)
    if args.compile:
        # flame compiles block by block (flame/models/parallelize_fla.py:369-403); the attention op
        # stays the registered custom op, the rest of a block is fused by the compiler
        for i, layer in enumerate(model.model.layers):
            model.model.layers[i] = torch.compile(layer)
    N = 8192
    lens = _lognormal_lengths(N, seed=0)
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    ids = torch.randint(0, cfg.vocab_size, (1, N), device=dev)
    settle_clocks(lambda: train_step(model, opt, ids, ids, cu_t, max(lens)), seconds=1.0)
    for _ in range(args.warmup):
        train_step(model, opt, ids, ids, cu_t, max(lens))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss, _ = train_step(model, opt, ids, ids, cu_t, max(lens))
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    n_noemb = model.num_parameters(exclude_embeddings=True)
    # flame's accounting (flame/tools/utils.py:39): 6*(N - N_emb) + 12*l*h*q*t FLOPs per token
    flops_tok = 6 * n_noemb + 12 * cfg.num_hidden_layers * cfg.num_heads * (cfg.hidden_size // cfg.num_heads) * N
    out = {
        "metric": "sba_340m_train_tokens_per_s", "value": round(N / (ms * 1e-3), 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg5: SBA-340M train step (24 layers, hidden 1024, 16x64 heads, MLP 2816, "
                               "vocab 32000), AdamW, bf16 autocast, one packed varlen row of 8192 tokens",
                   "params_M": round(model.num_parameters() / 1e6, 1), "n_docs": len(lens), "max_len": max(lens),
                   "compiled_blocks": bool(args.compile)},
        "final_loss": round(float(loss), 4),
        "mfu_flame_convention": round(flops_tok * N / (ms * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4),
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg2", choices=["cfg2", "cfg3", "cfg4", "cfg5", "short", "copy", "d256"])
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16"],
                    help="element type of the operator workloads (f16: the same kernels compiled for float16; "
                         "BASELINE.json's configurations are bf16, the default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--carries", default="kept", choices=["kept", "default"],
                    help="kept: the forward keeps its carry tables whatever their size (the kernels as such); default: the "
                         "operator's own rule, which above its workspace budget (256 MiB) keeps nothing and lets the "
                         "backward rebuild them (cfg4: 270 MB)")
    ap.add_argument("--autograd-thread", default="off", choices=["off", "on"],
                    help="off (default): torch.autograd.set_multithreading_enabled(False), the backward is issued from the "
                         "calling thread; on: PyTorch's default worker thread per device")
    ap.add_argument("--compile", action="store_true",
                    help="cfg5 only: torch.compile every block, as flame does with --training.compile")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the operator has no cross-GPU part "
                         "(heads and documents shard with no exchange); run with --gpus 1")

    import torch
    from flame_amd import sb_attn, sb_attn_varlen
    from flame_amd.stickbreaking_attention import profiling

    dev = torch.device("cuda:0")
    if args.autograd_thread == "off":
        # The backward runs in the calling thread instead of autograd's per-device worker: a forward + backward of the
        # operator then costs the host about 80 us instead of 160-200, which on a box with a slow host is the
        # difference between timing the kernels and timing Python.  Same graph, same kernels, same results.
        torch.autograd.set_multithreading_enabled(False)
    if args.workload == "cfg5":
        return bench_model(args, dev)
    if args.workload == "copy":
        # plain 256 MiB device copy: the known-size kernel that the FETCH_SIZE / WRITE_SIZE
        # counters of a profile are scaled by
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "copy", "bytes_read": 256 << 20, "bytes_written": 256 << 20}))
        return
    desc, (q, k, v, do, cu, max_len), pairs, tokens, D, H = make_workload(args.workload, dev, args.dtype)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    from flame_amd import _lib
    if args.carries == "kept":
        _lib.set_workspace_budget(float("inf"))

    def step():
        if cu is None:
            o, rem = sb_attn(q, k, v)
        else:
            o, rem = sb_attn_varlen(q, k, v, cu, max_len)
        # the three gradients straight from the backward (no accumulation nodes between the operator and the leaves)
        q.grad, k.grad, v.grad = torch.autograd.grad([o], [q, k, v], [do])
        return o, rem

    settle_clocks(step)
    for _ in range(args.warmup):
        step()
    # Kernel durations come from HIP events on the launch stream inside the timed region, on a
    # few evenly spaced steps: an event record stalls the queue for a few microseconds, and five of
    # them on every step would cost this workload more than a tenth of its time.
    every = max(1, args.steps // KERNEL_TIMING_SAMPLES)
    timer = profiling.KernelTimer(every=every)
    profiling.install(timer)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        timer.next_step()
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    profiling.install(None)

    ms = dt * 1e3 / args.steps
    f_fb = 12.0 * D * pairs
    tflops = f_fb / (ms * 1e-3) / 1e12
    kern = {name: sum(v_) / len(v_) for name, v_ in timer.durations_ms().items()}
    # algorithmic FLOPs per launch: each of the three kernels carries two of the six
    # counted products (4*d*P); recomputed products are not counted
    per_kernel_flops = 4.0 * D * pairs
    dom = max(kern, key=kern.get)
    desc["carries"] = "recomputed in the backward" if "bwd_carries_dq" in kern else "kept from the forward"
    achieved = per_kernel_flops / (kern[dom] * 1e-3) / 1e12
    out = {
        "metric": "sb_attn_fwd_bwd_tflops", "value": round(tflops, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic", "config": desc,
        "pct_of_bf16_mfma_peak": round(100 * tflops / BF16_MFMA_PEAK_TFLOPS, 2),
        "tokens_per_s": round(tokens / (ms * 1e-3), 1),
        "flops_convention": "12*d*P, P = allowed (query,key) pairs; recompute not counted",
        "kernel_ms": {n: round(t, 4) for n, t in kern.items()},
        "kernel_timing": f"HIP events on the launch stream, every {every}th step of the timed region",
        "fwd_tflops": round(4.0 * D * pairs / (kern.get("fwd", float("nan")) * 1e-3) / 1e12, 2),
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2),
                     "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / BF16_MFMA_PEAK_TFLOPS, 4),
                     "traffic": profiled_hbm_bytes(args.workload, dom),
                     "traffic_source": f"profiles/sba_{args.workload}_hbm_traffic.txt (rocprofv3 --pmc, not measured by this run)"},
    }
    if args.workload == "short":
        # algorithmic bytes per launch: q, k, v (+ dO) read once, the outputs written once (bf16), rem and the
        # carries not counted: forward 4 tensors, dQ pass 5, dK/dV pass 6
        unit = tokens * H * D * 2
        nbytes = {"fwd": 4 * unit, "bwd_dq": 5 * unit, "bwd_dkv": 6 * unit}
        gbs = {n: nbytes[n] / (kern[n] * 1e-3) / 1e9 for n in kern if n in nbytes}
        out["roofline"] = {"bound": "hbm", "kernel": dom, "achieved": round(gbs[dom], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(gbs[dom] / HBM_PEAK_GBS, 4), "traffic": None,
                           "per_kernel_GBps": {n: round(x, 1) for n, x in gbs.items()},
                           "step_GBps": round(15 * unit / (ms * 1e-3) / 1e9, 1)}
    fl = issue_floors(args.workload, dom, pairs) if dom in KERNEL_COLUMN else None
    if fl is not None:
        # what the dominant kernel could reach if only instruction issue limited it (MFMA time + vector time): with
        # the instructions it executes today, and with the fewest the algorithm needs
        at = lambda ms_: round(per_kernel_flops / (ms_ * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4)
        out["issue_floor"] = {"kernel": dom, "measured_ms": round(kern[dom], 4),
                              "floor_ms": round(fl["present_counts"], 4),
                              "frac_of_floor_rate": round(fl["present_counts"] / kern[dom], 3),
                              "frac_of_mfma_peak_at_floor": at(fl["present_counts"]),
                              "minimum_counts_floor_ms": round(fl["minimum_counts"], 4),
                              "frac_of_mfma_peak_at_minimum_counts": at(fl["minimum_counts"]),
                              "cycles_per_instruction": ISSUE_CYCLES, "clock_ghz": MIXED_CLOCK_GHZ,
                              "source": f"instruction counts from profiles/sba_{args.workload}_shader_counters.txt, "
                                        "issue rates from profiles/gfx950_issue_rates.txt"}
        every_kernel = [issue_floors(args.workload, n, pairs) if n in KERNEL_COLUMN else None for n in kern]
        if all(every_kernel):
            # the same two ceilings for the whole step (the three kernels one after the other)
            for which in ("present_counts", "minimum_counts"):
                total = sum(f[which] for f in every_kernel)
                out["issue_floor"][f"step_pct_of_mfma_peak_at_{which}"] = round(
                    100 * f_fb / (total * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 1)
    # (the CPU leg is defined for BASELINE's configurations, which are bf16)
    if not args.no_cpu_baseline and args.workload not in ("short", "d256") and args.dtype == "bf16":
        out["cpu_baseline"] = cpu_baseline(args.workload)
        o, rem = step()          # the timed tensors once more, for the check below
        out["parity_sample"] = parity_sample(args.workload, q, k, v, do, cu, o, rem)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
