"""Benchmark of the chunked delta-rule scan on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload gdn_chunk|kda_chunk|deltanet_varlen|deltanet_fp32|gdn_dk256|decode|...]

Default workload: Gated DeltaNet chunked forward+backward at B=8, H=16, T=4096, dk=dv=128,
bf16 q/k/v/dO, fp32 beta/g, chunk 64 (benchmark configuration 2).  One "step" is one forward
plus one backward pass through the public ops (``gated_delta_rule_chunkwise`` + autograd),
inputs resident in HBM.  Prints ONE JSON line; ``value`` is tokens/s = B*T / step time.

Before the W warm-up steps the workload runs untimed for ``--clock-warmup-seconds`` (default 2): the
shader clock of an idle MI355X sits near 100 MHz and takes about two seconds of load to reach
its 2.4 GHz, so W = 5 steps (5 ms) followed by 20 timed ones would time the ramp, not the
kernels.  The JSON line says how long and how many steps that was (``clock_warmup``); the
timed region is still exactly K steps.

``roofline`` describes the kernel with the largest share of the step, timed with HIP events
recorded by the library on the launch stream during the timed steps; ``achieved`` is that
kernel's algorithmic FLOP/s (or bytes/s).  ``cpu_baseline`` times the CPU restatement of the
same chunk algorithm (torch, all host cores) on a bounded sample of the workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

C = 64
PEAK_BF16 = 2500.0  # TFLOP/s, dense bf16 MFMA, MI355X
PEAK_HBM = 8000.0   # GB/s
PEAK_FP32_MFMA = 157.3  # TFLOP/s
CLOCK_WARMUP_S = 2.0    # set from --clock-warmup-seconds


def clock_warmup(torch, fn, seconds=None):
    """Runs fn untimed until `seconds` of wall clock have passed (the GPU's clocks leave their idle state); returns
    the number of calls."""
    seconds = CLOCK_WARMUP_S if seconds is None else min(seconds, CLOCK_WARMUP_S)
    n = 0
    if seconds <= 0:
        return n
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
        n += 8
    return n

def sources_sha256(files):
    """Hash of the named kernel sources, so that counter figures are only quoted for the code they were taken on."""
    import hashlib
    h = hashlib.sha256()
    for f in sorted(files):
        h.update(f.encode())
        with open(os.path.join(ROOT, "linearnexus_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs recorded in
    profiles/traffic.json, and where the figure comes from; (None, reason) when the kernel sources have changed
    since those runs."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as fh:
            rec = json.load(fh)
    except (OSError, ValueError):
        return None, "profiles/traffic.json missing"
    reason = "not measured"
    for entry in rec.get("measurements", []):
        if kernel in entry.get("workloads", {}).get(workload, {}):
            try:
                same = entry.get("sources_sha256") == sources_sha256(entry.get("sources", []))
            except OSError:
                same = False
            if same:
                return entry["workloads"][workload][kernel], f"profiles/traffic.json, commit {entry.get('commit')}"
            reason = f"profiles/traffic.json entry of commit {entry.get('commit')} predates the current kernel sources"
    return None, reason


def chunk_flops(dk, dv, direct=False):
    """Dense-product FLOPs per (batch, head, chunk) that each kernel performs.  In the WY split the forward
    terms add up to F_chunk = 2C^2(3dk+2dv) + 6C*dk*dv and the backward terms to 2*F_chunk; `direct` is the split of
    the kernels for 2-byte inputs with dk <= 128 and no per-channel gate."""
    cc, cd = 2 * C * C, 2 * C * dk * dv
    if direct:
        return {
            "chunk_prepare": 2 * cc * dk,                     # K K^T, Q K^T
            "chunk_scan": 3 * cd + 2 * cc * dv,               # K S, Q S, Tm R, Pm D, K^T D
            "bwd_scan": 3 * cd + 2 * cc * dv,                 # K dS, Pm^T dO, Tm^T dD, Q^T dO, K^T dY
            "bwd_chunk": 3 * cd + 2 * cc * dv + 4 * cc * dk,  # dO S^T, dR S^T, D dS^T, dO D^T, dR D^T, dPe K, dXa K, dPe^T Q, dXe^T K
        }
    return {
        "chunk_prepare": cc * (3 * dk + dv),          # K K^T, Q K^T, Tm(beta K), Tm(beta V)
        "chunk_scan": 2 * cd,                         # W S, K^T D
        "chunk_output": cd + cc * dv,                 # Q S, P D
        "bwd_local": cc * dv,                         # P^T dO
        "bwd_scan": 3 * cd,                           # K dS, Q^T dO, W^T dD
        "bwd_dqk": cc * dv + 3 * cd + 2 * cc * dk,    # dO D^T, dO S^T, dD S^T, D dS^T, dPe K, dPe^T Q
        "bwd_wy": cc * (4 * dk + 2 * dv),             # Tm^T dW, Tm^T dD, dBw W^T + dBu U^T, K K^T, Y K
    }


def make_cu_seqlens(seed, nseq, total, lo, hi, max_tries=1000):
    """cu_seqlens of `nseq` sequence lengths uniform in [lo, hi] that sum to `total` (configuration 5)."""
    import numpy as np
    rng = np.random.default_rng(seed)
    for _ in range(max_tries):
        lens = rng.integers(lo, hi + 1, size=nseq).astype(np.int64)
        lens = np.floor(lens * (total / lens.sum())).astype(np.int64)
        lens[-1] += total - lens.sum()
        if lens.min() >= lo and lens.max() <= hi:
            return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    raise RuntimeError("could not draw sequence lengths in range")


def make_gdn_inputs(torch, B, H, T, d, seed, device, dv=None):
    dv = dv or d
    gen = torch.Generator(device="cpu").manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    nrm = lambda x: x / (x.norm(dim=-1, keepdim=True) + 1e-6)
    q, k = nrm(rn(B, H, T, d)), nrm(rn(B, H, T, d))
    v = rn(B, H, T, dv)
    beta = torch.sigmoid(rn(B, H, T))
    g = -torch.nn.functional.softplus(rn(B, H, T)) * 0.1
    dO = rn(B, H, T, dv)
    return {n: t.to(device) for n, t in dict(q=q, k=k, v=v, beta=beta, g=g, dO=dO).items()}


def cpu_baseline_chunk(torch, B, H, T, d, seed):
    """fwd+bwd of the CPU restatement (chunk form + autograd) on a bounded sample: B_s batch rows."""
    from oracle import torch_ref as tr

    threads = torch.get_num_threads()
    Bs, passes = B, 2  # the whole workload, twice: 10-15 s of CPU work on 16 cores
    x = make_gdn_inputs(torch, Bs, H, T, d, seed, "cpu")

    def run(xs):
        inp = {"q": xs["q"], "k": xs["k"], "v": xs["v"], "beta": xs["beta"], "g": xs["g"], "initial_state": None}
        tr.grads(tr.chunkwise, inp, xs["dO"], None, use_qk_l2norm=False)

    run({n: t[:1, :2] for n, t in x.items()})  # warm-up
    t0 = time.perf_counter()
    for _ in range(passes):
        run(x)
    dt = (time.perf_counter() - t0) / passes
    return {"value": Bs * T / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"B={Bs} of {B} batch rows, H={H}, T={T}, d={d}, fp32, {passes} timed passes of {dt:.1f} s each"}


CHUNK_CONFIGS = {
    # name: (variant, B, H, T, d, packed sequences, random S0, backward)
    "gdn_chunk": ("gated", 8, 16, 4096, 128, 0, False, True),        # configuration 2 (headline)
    # configuration 2 through the reference's default, use_qk_l2norm=True, on q and k that are not normalised
    "gdn_chunk_l2norm": ("gated", 8, 16, 4096, 128, 0, False, True),
    "kda_chunk": ("kda", 4, 16, 8192, 128, 0, True, True),           # configuration 3
    # configuration 3 from the block's raw gate projection: kda_gate's activation inside the chunk kernels
    # (kda_chunkwise_raw_gate), against the same step behind the stand-alone gate kernels (kda_chunk_gate_kernels)
    "kda_chunk_raw_gate": ("kda", 4, 16, 8192, 128, 0, True, True),
    "kda_chunk_gate_kernels": ("kda", 4, 16, 8192, 128, 0, True, True),
    "deltanet_varlen": ("delta", 1, 32, 32768, 128, 8, False, True),  # configuration 5
    "deltanet_fp32": ("delta32", 2, 4, 512, 64, 0, False, False),     # configuration 1 (forward only)
    # head shape of the reference's Gated DeltaNet presets (models.py:142-143: head_dim 256, expand_v 2), 2048 wide
    "gdn_dk256": ("gated", 8, 8, 4096, (256, 512), 0, False, True),
    # fp32 inputs (the reference's models run fp32 unless told otherwise): configuration 2's shape and the presets'
    "gdn_chunk_fp32": ("gated32", 8, 16, 4096, 128, 0, False, True),
    "gdn_dk256_fp32": ("gated32", 8, 8, 4096, (256, 512), 0, False, True),
    "kda_chunk_fp32": ("kda32", 4, 16, 8192, 128, 0, True, True),
}


def bench_chunk(args, torch, la, _lib, name):
    variant, B, H, T, d, nseq, with_s0, backward = CHUNK_CONFIGS[name]
    dev = "cuda:0"
    l2norm = name.endswith("_l2norm")
    seed = {"deltanet_fp32": 1, "gdn_chunk": 2, "gdn_chunk_l2norm": 2, "kda_chunk": 3, "kda_chunk_raw_gate": 3,
            "kda_chunk_gate_kernels": 3, "deltanet_varlen": 5, "gdn_dk256": 6,
            "gdn_chunk_fp32": 2, "gdn_dk256_fp32": 6, "kda_chunk_fp32": 3}[name]
    fp32 = variant.endswith("32")
    variant = variant[:-2] if fp32 else variant
    d, dv = d if isinstance(d, tuple) else (d, d)
    x = make_gdn_inputs(torch, B, H, T, d, seed, dev, dv)
    dt = torch.float32 if fp32 else torch.bfloat16
    if l2norm:  # rows of length about sqrt(d), normalised inside the op
        x["q"], x["k"] = x["q"] * d ** 0.5, x["k"] * d ** 0.5
    q, k, v, dO = (x[n].to(dt) for n in ("q", "k", "v", "dO"))
    beta, g = x["beta"], x["g"]
    gen = torch.Generator(device="cpu").manual_seed(seed + 100)
    raw_gate = name in ("kda_chunk_raw_gate", "kda_chunk_gate_kernels")
    if variant == "kda":
        g = (-torch.nn.functional.softplus(torch.randn(B, H, T, d, generator=gen)) * 0.05).to(dev)
    if raw_gate:  # g = -exp(A_log) softplus(raw + bias) with A_log = log 0.05, bias = 0: the same decays as configuration 3
        import math
        g = None
        raw = torch.randn(B, H, T, d, generator=gen).to(dev).to(dt)  # head-first like q, k, v here: no layout copies in either form
        A_log = torch.full((H,), math.log(0.05), device=dev)
        g_bias = torch.zeros(H * d, device=dev)
    cu = None
    nstate = B
    if nseq:
        cu_np = make_cu_seqlens(seed, nseq, T, 1024, 8192)
        cu = torch.from_numpy(cu_np).to(dev)
        nstate = nseq
    s0 = (torch.randn(nstate, H, d, dv, generator=gen) * 0.02).to(dev) if (with_s0 or nseq) else None
    leaves = [q, k, v, beta] + ([g] if variant in ("gated", "kda") and not raw_gate else []) + ([s0] if s0 is not None else [])
    if raw_gate:
        leaves += [raw, A_log, g_bias]
    if backward:
        for t in leaves:
            t.requires_grad_(True)

    def forward():
        if variant == "gated":
            return la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, s0, 64, l2norm)
        if name == "kda_chunk_raw_gate":
            return la.kda_chunkwise_raw_gate(q, k, v, raw, beta, A_log, g_bias, None, s0, 64, False)
        if name == "kda_chunk_gate_kernels":  # every (batch, head) as a one-head batch row of the gate kernel (A_log is uniform here)
            ga, _ = la.kda_gate(raw.view(B * H, T, d), A_log[:1], d, g_bias[:d], out_dtype=torch.float32)
            return la.kda_chunkwise(q, k, v, ga.view(B, H, T, d), beta, None, s0, 64, False)
        if variant == "kda":
            return la.kda_chunkwise(q, k, v, g, beta, None, s0, 64, False)
        return la.delta_rule_chunkwise(q, k, v, beta, s0, cu_seqlens=cu)

    def step():
        for t in leaves:
            t.grad = None
        o, S = forward()
        if backward:
            o.backward(dO.to(o.dtype))

    n_clock = clock_warmup(torch, step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    per_kernel = {}
    t0 = time.perf_counter()
    for i in range(args.steps):
        step()
        if (i + 1) % 512 == 0:  # the library keeps a bounded number of event marks
            for kn, ms in _lib.profile_read():
                per_kernel.setdefault(kn, []).append(ms)
    torch.cuda.synchronize()
    dtm = (time.perf_counter() - t0) / args.steps
    for kn, ms in _lib.profile_read():
        per_kernel.setdefault(kn, []).append(ms)
    _lib.profile_enable(False)

    # the same forward without gradients (prefill / inference): forward_only is set, nothing is saved
    fwd_only_ms = float("nan")
    if not args.no_forward_only:
        with torch.no_grad():
            clock_warmup(torch, forward, 0.25)
            for _ in range(2):
                forward()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(args.steps):
                forward()
            torch.cuda.synchronize()
            fwd_only_ms = (time.perf_counter() - t1) / args.steps * 1e3

    if nseq:
        nchunks = H * int(sum(-(-int(l) // C) for l in (cu_np[1:] - cu_np[:-1])))
    else:
        nchunks = B * H * (-(-T // C))
    avg = {n: sum(v_) / len(v_) for n, v_ in per_kernel.items()}
    fl = chunk_flops(d, dv, direct="bwd_chunk" in avg)
    if "chunk_output" not in avg and "chunk_output" in fl:  # 2-byte inputs: the scan kernel also forms the outputs
        fl["chunk_scan"] += fl.pop("chunk_output")
    if "bwd_local" not in avg and "bwd_local" in fl:     # ... and the backward scan the chunk-local part of dD
        fl["bwd_scan"] += fl.pop("bwd_local")
    dom = max(avg, key=avg.get)
    achieved = fl[dom] * nchunks / (avg[dom] * 1e-3) / 1e12
    peak = PEAK_FP32_MFMA if fp32 else PEAK_BF16
    total_fl = (3 if backward else 1) * (2 * C * C * (3 * d + 2 * dv) + 6 * C * d * dv) * nchunks
    tr, tr_src = measured_traffic(name, dom)
    out = {
        "metric": "delta-rule chunk fwd+bwd tokens/s, % MFMA peak; decode-step HBM GB/s",
        "value": B * T / dtm, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dtm * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if fp32 else "bf16", "data": "synthetic",
        "clock_warmup": {"seconds": CLOCK_WARMUP_S, "steps": n_clock,
                         "why": "untimed steps before the W warm-up steps: the idle shader clock (about 100 MHz) needs about 2 s of load to reach 2.4 GHz"},
        "config": {"workload": name + ("_fwd_bwd" if backward else "_fwd"), "variant": variant, "B": B, "H": H, "T": T,
                   "dk": d, "dv": dv, "chunk": C, "packed_sequences": nseq, "initial_state": s0 is not None,
                   "use_qk_l2norm": l2norm,
                   "inputs": ("q,k rows of length sqrt(d), normalised inside the op" if l2norm else "q,k pre-normalised") + "; fp32 beta/g"},
        "tflops_algorithmic": total_fl / dtm / 1e12,
        "mfma_peak_frac": total_fl / dtm / 1e12 / peak,
        "kernel_ms": {n: round(t, 4) for n, t in avg.items()},
        "forward_only_ms": None if fwd_only_ms != fwd_only_ms else round(fwd_only_ms, 4),
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                     "frac": achieved / peak, "traffic": tr, "traffic_source": tr_src},
    }
    if tr:  # the same kernel against the HBM roof, from its measured traffic
        out["roofline_hbm_measured"] = {"kernel": dom, "achieved": tr / (avg[dom] * 1e-3) / 1e9, "peak": PEAK_HBM,
                                        "unit": "GB/s", "frac": tr / (avg[dom] * 1e-3) / 1e9 / PEAK_HBM}
    # The whole step against the HBM roof: every input read once and every output written once (no intermediates),
    # beside the traffic the kernels were measured to move (None when a kernel has no current entry).
    es, n = (4 if fp32 else 2), B * H * T
    eo = 4 if variant == "kda" else es  # kda_chunkwise returns fp32 (kda.py:655), so o and dO are fp32
    gate_el = {"delta": 0, "gated": 1, "kda": d}[variant]
    nstate = (nseq or B) * H * d * dv * 4
    alg = n * (es * (2 * d + dv) + eo * dv + 4 * (1 + gate_el)) + nstate * (2 if s0 is not None else 1)
    if backward:
        alg += n * (es * (2 * d + dv) + eo * dv + es * (2 * d + dv) + 4 * 2 * (1 + gate_el)) + (nstate if s0 is not None else 0)
    per = [measured_traffic(name, k_)[0] for k_ in avg]
    moved = sum(per) if all(per) else None
    out["step_hbm"] = {"algorithmic_bytes": alg, "algorithmic_GBps": alg / dtm / 1e9, "measured_bytes": moved,
                       "measured_GBps": None if moved is None else moved / dtm / 1e9,
                       "frac_of_peak_measured": None if moved is None else moved / dtm / 1e9 / PEAK_HBM, "peak": PEAK_HBM}
    return out, (B, H, T, d)


def bench_hbm_streams(torch, steps):
    """What plain streaming passes over 2 GiB sustain on this GPU: a read (sum), a write (fill) and a copy, as library
    kernels.  The byte-bound kernels are judged against these as well as against the 8 TB/s of the data sheet: reads and
    writes share the bus, and writes sustain markedly less than reads."""
    n = (2 << 30) // 4
    x = torch.ones(n, dtype=torch.float32, device="cuda:0")
    y = torch.empty_like(x)
    ops = {"read (sum)": (lambda: x.sum(), 4 * n), "write (fill_)": (lambda: y.fill_(1.0), 4 * n),
           "copy (copy_)": (lambda: y.copy_(x), 8 * n)}
    clock_warmup(torch, ops["copy (copy_)"][0], CLOCK_WARMUP_S)
    res = {}
    for name, (fn, nbytes) in ops.items():
        for _ in range(5):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        res[name] = {"ms": round(ms, 4), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac_of_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM, 3)}
    return {"metric": "streaming passes over 2 GiB: GB/s", "value": res["read (sum)"]["GBps"], "unit": "GB/s", "n_gpus": 1,
            "steps": steps, "warmup": 5, "ms_per_step": res["read (sum)"]["ms"], "higher_is_better": True, "vs_baseline": None,
            "dtype": "f32", "data": "synthetic", "config": {"workload": "hbm_streams", "bytes": 4 * n}, "streams": res}


def bench_decode(args, torch, la, _lib, steps=None):
    """Gated DeltaNet decode step at B=256, H=32, dk=dv=128: fp32 state updated in place.  The timed loop replays the
    step as a captured HIP graph (linearnexus_amd.decode.DecodeGraph -- the per-token loop of generate.py:243-271 with
    one host call per token); the same steps through one eager op call each are reported beside it."""
    from linearnexus_amd.decode import DecodeGraph
    B, H, d = 256, 32, 128
    dev = "cuda:0"
    gen = torch.Generator(device="cpu").manual_seed(4)
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    nrm = lambda x: x / (x.norm(dim=-1, keepdim=True) + 1e-6)
    S = (rn(B, H, d, d) * 0.02).to(dev)
    dg = DecodeGraph("gated", B, H, d, d, layers=1, dtype=torch.bfloat16, use_qk_l2norm=False, states=[S])
    dg.step(nrm(rn(B, H, d)).to(dev).bfloat16(), nrm(rn(B, H, d)).to(dev).bfloat16(), rn(B, H, d).to(dev).bfloat16(),
            torch.sigmoid(rn(B, H)).to(dev), (-torch.nn.functional.softplus(rn(B, H)) * 0.1).to(dev))
    steps = steps or 1000

    def timed(fn):
        clock_warmup(torch, fn, 0.5)
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        _lib.profile_enable(True)
        kern = []
        t0 = time.perf_counter()
        for i in range(steps):
            fn()
            if (i + 1) % 2048 == 0:
                kern += [ms for _, ms in _lib.profile_read()]
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        kern += [ms for _, ms in _lib.profile_read()]
        _lib.profile_enable(False)
        return dt, kern

    dt_eager, kern = timed(dg._run)     # per-kernel HIP events are recorded on eager launches only
    dt, _ = timed(dg.replay)
    nbytes = 2 * S.numel() * 4 + 4 * B * H * d * 2 + 2 * B * H * 4
    kms = sum(kern) / len(kern)
    tr, tr_src = measured_traffic("decode", "decode_step")
    return {
        "workload": "gated_deltanet_decode_step", "B": B, "H": H, "dk": d, "dv": d, "steps": steps, "driver": "captured graph replay",
        "ms_per_step": dt * 1e3, "tokens_per_s": B / dt, "bytes_per_step": nbytes,
        "wall_frac_of_hbm_peak": nbytes / dt / 1e9 / PEAK_HBM, "eager_ms_per_step": dt_eager * 1e3,
        "roofline": {"bound": "hbm", "kernel": "decode_step", "achieved": nbytes / (kms * 1e-3) / 1e9, "peak": PEAK_HBM,
                     "unit": "GB/s", "frac": nbytes / (kms * 1e-3) / 1e9 / PEAK_HBM,
                     "traffic": tr, "traffic_source": tr_src},
    }


def bench_conv(torch, la, _lib, steps, warmup):
    """Causal depthwise conv (K=4) + SiLU over the q|k|v projections of config 2's layer: [B8, T4096, D6144] bf16,
    forward + backward.  Algorithmic bytes: x in, y out; x, dy in, dx out (weights are 100 KB)."""
    B, T, D, K = 8, 4096, 6144, 4
    gen = torch.Generator(device="cpu").manual_seed(6)
    x = torch.randn(B, T, D, generator=gen).to("cuda:0").bfloat16().requires_grad_(True)
    dy = torch.randn(B, T, D, generator=gen).to("cuda:0").bfloat16()
    w = (torch.randn(K, D, generator=gen) * 0.3).to("cuda:0").requires_grad_(True)

    def step():
        x.grad = w.grad = None
        y, _ = la.depthwise_conv1d_causal(x, w, None, activation="silu")
        y.backward(dy)

    clock_warmup(torch, step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    marks = _lib.profile_read()
    _lib.profile_enable(False)
    avg = {n: sum(ms for m, ms in marks if m == n) / max(1, sum(1 for m, _ in marks if m == n)) for n in ("conv1d_fwd", "conv1d_bwd")}
    nb = {"conv1d_fwd": 2 * B * T * D * 2, "conv1d_bwd": 3 * B * T * D * 2}
    dom = "conv1d_bwd"
    ach = nb[dom] / (avg[dom] * 1e-3) / 1e9
    return {"metric": "causal depthwise conv + SiLU fwd+bwd tokens/s", "value": B * T / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "conv1d_silu_fwd_bwd", "B": B, "T": T, "D": D, "K": K},
            "kernel_ms": {n: round(v, 4) for n, v in avg.items()},
            "roofline": {"bound": "hbm", "kernel": dom, "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": ach / PEAK_HBM, "traffic": None},
            "roofline_fwd": {"bound": "hbm", "kernel": "conv1d_fwd", "achieved": nb["conv1d_fwd"] / (avg["conv1d_fwd"] * 1e-3) / 1e9,
                             "peak": PEAK_HBM, "unit": "GB/s", "frac": nb["conv1d_fwd"] / (avg["conv1d_fwd"] * 1e-3) / 1e9 / PEAK_HBM}}


def bench_dplr_step(torch, la, _lib, steps):
    """RWKV-7 DPLR decode step at config 4's shape (B=256, H=32, dk=dv=128), fp32 state updated in place.
    Algorithmic bytes: the state read and written once, five bf16 dk-vectors, gk fp32, v in, o out."""
    B, H, d = 256, 32, 128
    gen = torch.Generator(device="cpu").manual_seed(7)
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    S = (rn(B, H, d, d) * 0.02).to("cuda:0")
    q, k, v = (rn(B, H, d).to("cuda:0").bfloat16() for _ in range(3))
    a, b = ((rn(B, H, d) * 0.1).to("cuda:0").bfloat16() for _ in range(2))
    gk = (-rn(B, H, d).abs() * 0.1).to("cuda:0")
    clock_warmup(torch, lambda: la.dplr_delta_rule_step(q, k, v, a, b, gk, S, inplace=True), 0.5)
    for _ in range(20):
        la.dplr_delta_rule_step(q, k, v, a, b, gk, S, inplace=True)
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        la.dplr_delta_rule_step(q, k, v, a, b, gk, S, inplace=True)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    kern = [ms for _, ms in _lib.profile_read()]
    _lib.profile_enable(False)
    nbytes = 2 * S.numel() * 4 + 6 * B * H * d * 2 + B * H * d * 4
    kms = sum(kern) / len(kern)
    ach = nbytes / (kms * 1e-3) / 1e9
    return {"metric": "DPLR decode-step HBM GB/s", "value": ach, "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": 20,
            "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic", "config": {"workload": "rwkv7_dplr_decode_step", "B": B, "H": H, "dk": d, "dv": d},
            "roofline": {"bound": "hbm", "kernel": "dplr_step", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": ach / PEAK_HBM, "traffic": None}}


def bench_dplr_train(torch, la, _lib, steps, warmup):
    """RWKV-7 DPLR scan forward + backward at B8 H16 T4096 dk=dv=64 bf16 (the block's head size 64): tokens/s, and the
    backward kernel against the HBM roofline.  Algorithmic bytes of the backward: every token's starting state is written
    to the segment tape and read back once (2 * 4 B per state element and token; the checkpoints add 1/64 of that), the
    token vectors are read three times (checkpoint sweep, tape sweep, reverse sweep), six fp32 gradients leave."""
    B, H, T, d = 8, 16, 4096, 64
    gen = torch.Generator(device="cpu").manual_seed(9)
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    q, k, v = (rn(B, H, T, d).to("cuda:0").bfloat16().requires_grad_(True) for _ in range(3))
    a, b = ((rn(B, H, T, d) * 0.1).to("cuda:0").bfloat16().requires_grad_(True) for _ in range(2))
    gk = (-rn(B, H, T, d).abs() * 0.1).to("cuda:0").requires_grad_(True)
    dO = rn(B, H, T, d).to("cuda:0").bfloat16()
    leaves = (q, k, v, a, b, gk)

    def step():
        for t in leaves:
            t.grad = None
        o, _ = la.dplr_delta_rule_recurrent(q, k, v, a, b, gk, d ** -0.5)
        o.backward(dO)
    clock_warmup(torch, step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    acc = {}
    for n, ms in _lib.profile_read():
        acc.setdefault(n, []).append(ms)
    _lib.profile_enable(False)
    avg = {n: sum(x) / len(x) for n, x in acc.items()}
    tok = B * H * T
    nbytes = tok * d * d * 4 * (2 + 1 / 64) + 3 * tok * (5 * d * 2 + d * 4 + d * 2) + tok * d * 2 + 6 * tok * d * 4
    ach = nbytes / (avg["dplr_bwd"] * 1e-3) / 1e9
    return {"metric": "DPLR scan fwd+bwd tokens/s", "value": B * T / dt, "unit": "tokens/s", "n_gpus": 1, "steps": steps,
            "warmup": warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": "rwkv7_dplr_scan_fwd_bwd", "B": B, "H": H, "T": T, "dk": d, "dv": d, "inputs": "bf16, fp32 gk"},
            "kernel_ms": {n: round(x, 4) for n, x in avg.items()},
            "roofline": {"bound": "hbm", "kernel": "dplr_bwd", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s",
                         "frac": ach / PEAK_HBM, "traffic": None}}


def bench_rmsnorm_gated(torch, la, _lib, steps, warmup):
    """Gated RMSNorm epilogue over config 2's outputs: x, gate [B8, T4096, H16, d128] bf16, forward + backward.
    Algorithmic bytes: x, gate in, y out; x, gate, dy in, dx, dgate out."""
    shape = (8, 4096, 16, 128)
    gen = torch.Generator(device="cpu").manual_seed(8)
    x, g, dy = (torch.randn(*shape, generator=gen).to("cuda:0").bfloat16() for _ in range(3))
    x.requires_grad_(True), g.requires_grad_(True)
    w = torch.ones(128, device="cuda:0", requires_grad=True)

    def step():
        x.grad = g.grad = w.grad = None
        la.rmsnorm_gated(x, g, w).backward(dy)

    clock_warmup(torch, step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    marks = _lib.profile_read()
    _lib.profile_enable(False)
    names = ("rmsnorm_gated_fwd", "rmsnorm_gated_bwd")
    avg = {n: sum(ms for m, ms in marks if m == n) / max(1, sum(1 for m, _ in marks if m == n)) for n in names}
    n_el = x.numel()
    nb = {"rmsnorm_gated_fwd": 3 * n_el * 2, "rmsnorm_gated_bwd": 5 * n_el * 2}
    roof = {n: {"bound": "hbm", "kernel": n, "achieved": nb[n] / (avg[n] * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s",
                "frac": nb[n] / (avg[n] * 1e-3) / 1e9 / PEAK_HBM, "traffic": None} for n in names}
    return {"metric": "gated RMSNorm fwd+bwd tokens/s", "value": shape[0] * shape[1] / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "rmsnorm_gated_fwd_bwd", "B": 8, "T": 4096, "H": 16, "d": 128},
            "kernel_ms": {n: round(v, 4) for n, v in avg.items()}, "roofline": roof["rmsnorm_gated_bwd"],
            "roofline_fwd": roof["rmsnorm_gated_fwd"]}


def bench_kda_gate(torch, la, _lib, steps, warmup):
    """KDA gate activation for config 3's gate tensor: raw gate [B4, T8192, H16*dk128] bf16 -> fp32 log-decay, forward
    + backward.  Algorithmic bytes: g (bf16) in, g_out (fp32) out; g, d_out (fp32) in, d_g (bf16) out."""
    B, T, H, dk = 4, 8192, 16, 128
    gen = torch.Generator(device="cpu").manual_seed(9)
    raw = torch.randn(B, T, H * dk, generator=gen).to("cuda:0").bfloat16().requires_grad_(True)
    dy = torch.randn(B, T, H, dk, generator=gen).to("cuda:0")
    A = torch.zeros(H, device="cuda:0", requires_grad=True)
    bias = torch.zeros(H * dk, device="cuda:0", requires_grad=True)

    def step():
        raw.grad = A.grad = bias.grad = None
        g, _ = la.kda_gate(raw, A, dk, bias, out_dtype=torch.float32)
        g.backward(dy)

    clock_warmup(torch, step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    marks = _lib.profile_read()
    _lib.profile_enable(False)
    names = ("kda_gate_fwd", "kda_gate_bwd")
    avg = {n: sum(ms for m, ms in marks if m == n) / max(1, sum(1 for m, _ in marks if m == n)) for n in names}
    n_el = raw.numel()
    nb = {"kda_gate_fwd": n_el * (2 + 4), "kda_gate_bwd": n_el * (2 + 4 + 2)}
    roof = {n: {"bound": "hbm", "kernel": n, "achieved": nb[n] / (avg[n] * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s",
                "frac": nb[n] / (avg[n] * 1e-3) / 1e9 / PEAK_HBM, "traffic": None} for n in names}
    return {"metric": "KDA gate activation fwd+bwd tokens/s", "value": B * T / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "kda_gate_fwd_bwd", "B": B, "T": T, "H": H, "dk": dk},
            "kernel_ms": {n: round(v, 4) for n, v in avg.items()}, "roofline": roof["kda_gate_bwd"],
            "roofline_fwd": roof["kda_gate_fwd"]}


def bench_decode_graph(torch, steps):
    """Host cost per generated token of a 24-layer Gated DeltaNet decode (B=1 and 8, H=32, d=128): the layers'
    steps replayed as one captured graph against one eager op call per layer."""
    from linearnexus_amd.decode import DecodeGraph
    res = []
    for B in (1, 8):
        H, d, L = 32, 128, 24
        dg = DecodeGraph("gated", B, H, d, d, layers=L)
        for i in range(L):
            dg.q[i].normal_(), dg.k[i].normal_(), dg.v[i].normal_(), dg.beta[i].fill_(0.5), dg.g[i].fill_(-0.1)
        us = {}
        for name, fn in (("graph", dg.replay), ("eager", dg._run)):
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            us[name] = (time.perf_counter() - t0) / steps * 1e6
        res.append({"B": B, "H": H, "dk": d, "dv": d, "layers": L, "graph_us_per_token": us["graph"],
                    "eager_us_per_token": us["eager"]})
    return res


def bench_prefill_long(torch, la, steps):
    """Forward only (prefill) of single long prompts, Gated DeltaNet bf16: one sequential chain per (head, value slab)
    against the segments-in-parallel form the ops pick for few long sequences (LNX_PREFILL_SEGMENTS=1 disables it)."""
    import os
    res = []
    for H, T, dk, dv in ((4, 65536, 128, 128), (16, 131072, 128, 128), (4, 32768, 256, 512)):
        gen = torch.Generator(device="cpu").manual_seed(7)
        rn = lambda *s_: torch.randn(*s_, generator=gen, dtype=torch.float32)
        nrm = lambda x: x / (x.norm(dim=-1, keepdim=True) + 1e-6)
        q, k = nrm(rn(1, H, T, dk)).to("cuda:0").bfloat16(), nrm(rn(1, H, T, dk)).to("cuda:0").bfloat16()
        v = rn(1, H, T, dv).to("cuda:0").bfloat16()
        beta = torch.sigmoid(rn(1, H, T)).to("cuda:0")
        g = (-torch.nn.functional.softplus(rn(1, H, T)) * 0.1).to("cuda:0")
        ms = {}
        for name, env in (("one_chain", "1"), ("segmented", None)):
            if env is None:
                os.environ.pop("LNX_PREFILL_SEGMENTS", None)
            else:
                os.environ["LNX_PREFILL_SEGMENTS"] = env
            with torch.no_grad():
                for _ in range(2):
                    la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
                torch.cuda.synchronize()
            ms[name] = (time.perf_counter() - t0) / steps * 1e3
        os.environ.pop("LNX_PREFILL_SEGMENTS", None)
        res.append({"B": 1, "H": H, "T": T, "dk": dk, "dv": dv, "one_chain_ms": ms["one_chain"],
                    "segmented_ms": ms["segmented"], "tokens_per_s": T / (ms["segmented"] * 1e-3)})
        del q, k, v, beta, g
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="gdn_chunk", choices=list(CHUNK_CONFIGS) + ["decode", "decode_graph", "conv", "dplr_decode", "dplr_train", "rmsnorm_gated", "kda_gate", "prefill_long", "hbm_streams"])
    ap.add_argument("--clock-warmup-seconds", type=float, default=2.0,
                    help="untimed run of the workload before the W warm-up steps, so that the timed steps see the GPU's "
                         "clocks at their loaded level and not on the way up from idle (0: none; counter runs use that)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-forward-only", action="store_true",
                    help="skip the extra forward-without-gradients timing (profiler runs: keeps the per-kernel averages to the differentiable step)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain 512 MiB device copy (known traffic) so that a counter run can be scaled")
    args = ap.parse_args()
    global CLOCK_WARMUP_S
    CLOCK_WARMUP_S = max(0.0, args.clock_warmup_seconds)
    if args.gpus != 1:
        print("bench.py measures one GPU only: the scan needs no collective and every figure here is "
              "single-GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    import linearnexus_amd as la
    from linearnexus_amd import _lib

    _lib.load()  # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (no GPU visible)", file=sys.stderr)
        sys.exit(2)

    if args.workload == "hbm_streams":
        print(json.dumps(bench_hbm_streams(torch, args.steps)))
        return
    if args.workload == "kda_gate":
        print(json.dumps(bench_kda_gate(torch, la, _lib, args.steps, args.warmup)))
        return
    if args.workload == "prefill_long":
        res = bench_prefill_long(torch, la, min(args.steps, 10))
        print(json.dumps({"metric": "single long prompt, forward only: tokens/s", "value": res[0]["tokens_per_s"],
                          "unit": "tokens/s", "n_gpus": 1, "steps": min(args.steps, 10), "warmup": 2,
                          "ms_per_step": res[0]["segmented_ms"], "higher_is_better": True, "vs_baseline": None,
                          "dtype": "bf16", "data": "synthetic", "config": {"workload": "gated_deltanet_prefill_long"},
                          "cases": res}))
        return
    if args.workload == "rmsnorm_gated":
        print(json.dumps(bench_rmsnorm_gated(torch, la, _lib, args.steps, args.warmup)))
        return
    if args.workload == "dplr_decode":
        print(json.dumps(bench_dplr_step(torch, la, _lib, max(args.steps, 500))))
        return
    if args.workload == "dplr_train":
        print(json.dumps(bench_dplr_train(torch, la, _lib, min(args.steps, 5), min(args.warmup, 2))))
        return
    if args.workload == "conv":
        print(json.dumps(bench_conv(torch, la, _lib, args.steps, args.warmup)))
        return
    if args.workload == "decode_graph":
        res = bench_decode_graph(torch, max(args.steps, 200))
        print(json.dumps({"metric": "decode host time per token, 24 layers", "value": res[0]["graph_us_per_token"],
                          "unit": "us/token", "n_gpus": 1, "steps": max(args.steps, 200), "warmup": 10,
                          "higher_is_better": False, "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                          "config": {"workload": "gated_deltanet_decode_graph"}, "cases": res}))
        return
    if args.workload == "decode":
        dec = bench_decode(args, torch, la, _lib, steps=max(args.steps, 100))
        out = {"metric": "delta-rule chunk fwd+bwd tokens/s, % MFMA peak; decode-step HBM GB/s",
               "value": dec["roofline"]["achieved"], "unit": "GB/s", "n_gpus": 1, "steps": dec["steps"],
               "warmup": 20, "ms_per_step": dec["ms_per_step"], "higher_is_better": True, "scaling": "weak",
               "vs_baseline": None, "dtype": "f32", "data": "synthetic",
               "config": {k_: dec[k_] for k_ in ("workload", "B", "H", "dk", "dv")}, "roofline": dec["roofline"]}
        print(json.dumps(out))
        return

    if args.calibrate:
        a = torch.empty(512 * 1024 * 1024 // 4, device="cuda:0").normal_()
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    cpu = None
    if not args.no_cpu_baseline and args.workload == "gdn_chunk":
        # the CPU leg first: the GPU legs then run back to back up to the end of the process
        _, cB, cH, cT, cd = CHUNK_CONFIGS["gdn_chunk"][:5]
        cpu = cpu_baseline_chunk(torch, cB, cH, cT, cd, 2)
    out, (B, H, T, d) = bench_chunk(args, torch, la, _lib, args.workload)
    if args.workload == "gdn_chunk":
        if not args.no_forward_only:
            # the same step through the reference's default use_qk_l2norm=True, on rows that are not normalised
            torch.cuda.empty_cache()
            l2, _ = bench_chunk(args, torch, la, _lib, "gdn_chunk_l2norm")
            out["use_qk_l2norm_true"] = {k_: l2[k_] for k_ in ("ms_per_step", "value", "unit", "kernel_ms", "forward_only_ms")}
            del l2
            torch.cuda.empty_cache()
        out["decode_step"] = bench_decode(args, torch, la, _lib)
    if cpu is not None:
        out["cpu_baseline"] = cpu
    print(json.dumps(out))


if __name__ == "__main__":
    main()
