#!/usr/bin/env python
"""Benchmark of the RFA kernel path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one causal forward + backward over one batch of synthetic input at the
configuration the headline metric is quoted on (seq 1024, batch 8, 8 heads,
head_dim 64, proj_dim 64, fp16), called through the C ABI (rfa_causal_forward_save +
rfa_causal_backward_saved, the pair RFA.apply(...).backward(...) runs) with all inputs resident in HBM.  One JSON line is printed:
the throughput of that step, the roofline of its dominant kernel (per-kernel
durations from HIP events recorded by the library around every launch), the same
step timed with the CPU oracle on the host cores, and -- as extra keys -- the decode,
cross-attention and feature-map figures.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

TRAFFIC_PROFILE = os.path.join("profiles", "bench_cfg2_hbm_traffic.md")


def _profile_traffic_bytes(*kernels):
    """Measured HBM bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE passes, counters scaled on
    the 512 MiB copy) of the named kernels, summed, read from the table of the tracked profile
    summary: `rfa::<name><...>` rows, first match per name.  None when a name has no row."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as fh:
            rows = [[c.strip() for c in ln.strip().strip("|").split("|")] for ln in fh if ln.startswith("| `rfa::")]
    except OSError:
        return None
    total = 0.0
    for name in kernels:
        hit = next((r for r in rows if r[0].strip("`").startswith("rfa::" + name)), None)
        if hit is None:
            return None
        total += float(hit[-1])
    return int(round(total * 1e6))


def _cpu_threads(torch):
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    return cores


def _event_time_ms(torch, fn, iters):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip decode / cross / feature-map figures")
    ap.add_argument("--skip", default="", help="comma-separated extras to leave out (decode_module: the per-token "
                    "module decode loop and its HIP graph)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every box of this build has one GPU and the path needs no "
                 "second one (sequences are independent); run with --gpus 1")

    import torch
    from oracle import rfa_oracle as O
    from rfa_amd import _lib, rfa_hip
    lib = _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream

    # ---------------------------------------------------------------- workload (config 2)
    T, B, H, d, D = 1024, 8, 8, 64, 64
    N, K = B * H, 2 * D
    q, k, v, g = O.make_qkv(T, B, H, d, seed=1234 + 2)
    W = O.make_w(d, D, H).half()
    cq, ck, cv, cg = (t.to(dev).contiguous() for t in (q, k, v, g))
    cW = W.to(dev)
    pq = rfa_hip.feature_map_forward(cq, cW, O.SCALE).view(T, N, K)
    pk = rfa_hip.feature_map_forward(ck, cW, O.SCALE).view(T, N, K)
    vv, gg = cv.view(T, N, d), cg.view(T, N, d)
    out = torch.empty_like(vv)
    dq, dk, dv = torch.empty_like(pq), torch.empty_like(pk), torch.empty_like(vv)
    fbytes = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
    bbytes = lib.rfa_causal_backward_workspace_bytes(T, N, K, d)
    ws = torch.empty(max(fbytes, bbytes, 1), dtype=torch.uint8, device=dev)
    p = lambda t: t.data_ptr()

    sbytes = lib.rfa_causal_saved_state_bytes(T, N, K, d)
    saved = torch.empty(max(sbytes, 1), dtype=torch.uint8, device=dev)

    def step():
        # what RFA.apply(...).backward(grad) runs: the forward hands its segment totals to the backward
        _lib.check(lib.rfa_causal_forward_save(p(pq), p(pk), p(vv), p(out), p(saved), sbytes, T, N, K, d,
                                               p(ws), fbytes, stream))
        _lib.check(lib.rfa_causal_backward_saved(p(pq), p(pk), p(vv), p(gg), p(out), p(saved), sbytes, p(dq), p(dk), p(dv),
                                                 T, N, K, d, p(ws), bbytes, stream))

    for _ in range(args.warmup):
        step()
    ms_per_step = _event_time_ms(torch, step, args.steps)          # the timed region: exactly K steps
    tokens = B * T
    value = tokens / (ms_per_step * 1e-3)

    # parity gate next to the timing (fp32 oracle on a slice of the batch: first 8 sequences)
    ns = 8
    ref = O.causal_forward_chunked(pq[:, :ns].float().cpu(), pk[:, :ns].float().cpu(), vv[:, :ns].float().cpu())
    rq, rk, rv = O.causal_backward_chunked(pq[:, :ns].float().cpu(), pk[:, :ns].float().cpu(),
                                           vv[:, :ns].float().cpu(), gg[:, :ns].float().cpu())
    rel = lambda a, b: ((a.float().cpu() - b).norm() / b.norm()).item()
    parity = {"out_max_abs": (out[:, :ns].float().cpu() - ref).abs().max().item(),
              "dq_rel": rel(dq[:, :ns], rq), "dk_rel": rel(dk[:, :ns], rk), "dv_rel": rel(dv[:, :ns], rv)}
    parity["ok"] = bool(parity["out_max_abs"] <= 2e-3 and max(parity["dq_rel"], parity["dk_rel"], parity["dv_rel"]) <= 1e-2)

    # ---------------------------------------------------------------- per-kernel durations
    _lib.check(lib.rfa_profile_reset())
    _lib.check(lib.rfa_profile_enable(1))
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    _lib.check(lib.rfa_profile_enable(0))
    totals = _lib.profile_totals()
    kern_us = {n: 1e3 * ms / c for n, (ms, c) in totals.items()}
    # algorithmic HBM bytes per launch: each kernel's inputs read once + outputs written once
    per_tok = {
        "k_segment_state": (K + d) * 2,
        "k_causal_fwd": (2 * K + d) * 2 + d * 2,
        "k_causal_bwd_dq": (2 * K + 3 * d) * 2 + K * 2 + 8,       # q, k, v, g, out in; dq out; den in, gz out
        "k_causal_bwd_dkdv": (2 * K + 2 * d) * 2 + 8 + (K + d) * 2,
        "k_sliced_bwd": (2 * K + 3 * d) * 2 + 4 + (2 * K + d) * 2,  # q, k, v, g, out, den in; dq, dk, dv out
    }
    nseg = lib.rfa_causal_num_segments(T, N, K, d)
    units = {n_: N * T for n_ in per_tok}
    units["k_segment_state"] = N * T * (nseg - 1) // max(nseg, 1)
    dominant = max((n_ for n_ in kern_us if n_ in per_tok), key=lambda n_: totals[n_][0])
    dom_bytes = per_tok[dominant] * units[dominant]
    achieved = dom_bytes / (kern_us[dominant] * 1e-6) / 1e9
    roofline = {"bound": "hbm", "kernel": dominant, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": _profile_traffic_bytes({"k_causal_fwd": "k_causal_fwd_pipe<128, 64, true>",
                                                   "k_segment_state": "k_segment_state<128, 64, 4, true, false>",
                                                   "k_sliced_bwd": "k_sliced_bwd<128, 64, 64>"}.get(dominant, dominant + "<")),
                "traffic_source": TRAFFIC_PROFILE + " (FETCH_SIZE + WRITE_SIZE of this kernel at this shape, a profile run "
                                  "of this file, not measured in this run)",
                "bytes_per_launch": dom_bytes, "avg_us": round(kern_us[dominant], 2),
                "kernels_us": {n_: round(u, 2) for n_, u in kern_us.items()},
                "step_algorithmic_bytes": 2176 * N * T,
                "step_frac_of_hbm": round(2176 * N * T / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    # ---------------------------------------------------------------- CPU baseline (oracle port)
    cpu_baseline = None
    if not args.no_cpu_baseline:
        cores = _cpu_threads(torch)
        bs = B                                                 # the whole batch: about 10 s of CPU work
        sq, sk = pq[:, :bs * H].float().cpu(), pk[:, :bs * H].float().cpu()
        sv, sg = vv[:, :bs * H].float().cpu(), gg[:, :bs * H].float().cpu()
        times = []
        for it in range(5):
            t0 = time.perf_counter()
            O.causal_forward_cumsum(sq, sk, sv)
            O.causal_backward_cumsum(sq, sk, sv, sg)
            times.append(time.perf_counter() - t0)
        tcpu = sorted(times[1:])[0] if len(times) > 1 else times[0]
        # the same step in the oracle's chunked form (no [T, N, K, d] temporaries): what a CPU
        # implementation that is not bound by those 2 GiB arrays reaches on the same threads
        ctimes = []
        for it in range(3):
            t0 = time.perf_counter()
            O.causal_forward_chunked(sq, sk, sv)
            O.causal_backward_chunked(sq, sk, sv, sg)
            ctimes.append(time.perf_counter() - t0)
        tchunk = min(ctimes[1:])
        cpu_baseline = {"value": round(bs * T / tcpu, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
                        "sample": f"causal fwd+bwd, cumulative-sum form (rfa.py:46-103) in fp32 torch-CPU on {bs} of "
                                  f"{B} batch entries (T={T}, {bs * H} sequences), 1 warm-up, best of 4",
                        "speedup": round(value / (bs * T / tcpu), 1),
                        "chunked_form_tokens_per_s": round(bs * T / tchunk, 1),
                        "chunked_form_speedup": round(value / (bs * T / tchunk), 1)}

    result = {
        "metric": "causal fwd+bwd tok/s @L=1024 fp16", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: RFA causal self-attention fwd+bwd, seq 1024, batch 8, 8 heads, "
                               "head_dim 64, proj_dim 64 (phi width 128), feature-level boundary RFA.apply",
                   "T": T, "B": B, "H": H, "head_dim": d, "proj_dim": D, "segments": nseg,
                   "backward": "one launch by state slices" if "k_sliced_bwd" in kern_us else "two sweeps over time segments",
                   "arithmetic": "fp16 operands and outputs, fp32 accumulation and state"},
        "parity": parity, "roofline": roofline, "cpu_baseline": cpu_baseline,
    }

    if not args.no_extras:
        skip = set(filter(None, args.skip.split(",")))
        if args.no_cpu_baseline:
            skip.add("cpu")
        result["extras"] = extras(torch, O, lib, _lib, rfa_hip, dev, stream, skip)
    print(json.dumps(result))


def extras(torch, O, lib, _lib, rfa_hip, dev, stream, skip=()):
    ex = {}
    p = lambda t: t.data_ptr()
    # ---- decode (config 4): B64 H16 d64 D64, 2048 steps after a 512-token prefill
    B, H, d, D, prefill, steps = 64, 16, 64, 64, 512, 2048
    N, K = B * H, 2 * D
    g = torch.Generator(device="cpu").manual_seed(1234 + 4)
    W = O.make_w(d, D, H).half().to(dev)
    unit = lambda t: t / t.norm(dim=-1, keepdim=True)
    pk_ = unit(torch.randn(prefill, B, H, d, generator=g)).half().to(dev)
    pv_ = torch.randn(prefill, B, H, d, generator=g).half().to(dev)
    s0, z0 = rfa_hip.cross_state(rfa_hip.feature_map_forward(pk_, W, O.SCALE), pv_)   # prefill state = sum over 512 tokens
    del pk_, pv_
    chunk = 256
    qs = unit(torch.randn(chunk, B, H, d, generator=g)).half().to(dev).repeat(steps // chunk, 1, 1, 1)
    ks = unit(torch.randn(chunk, B, H, d, generator=g)).half().to(dev).repeat(steps // chunk, 1, 1, 1)
    vs = torch.randn(chunk, B, H, d, generator=g).half().to(dev).repeat(steps // chunk, 1, 1, 1)
    outs = torch.empty_like(vs)
    s, z = s0.clone(), z0.clone()

    # (1) What a decoder does: the rows of a step are written on the device (by the projection
    # GEMMs) just before the step.  The 2048 steps run as 32 calls of 64 steps, each preceded by an
    # (untimed) elementwise pass that rewrites that call's q, k, v rows.  This is the quoted figure.
    def run_decode(n_steps, off=0):
        _lib.check(lib.rfa_incremental_fused(p(qs) + off, p(ks) + off, p(vs) + off, p(W), O.SCALE, p(s), p(z),
                                             p(outs) + off, n_steps, B, H, D, d, stream))
    run_decode(steps)
    s.copy_(s0); z.copy_(z0)
    step_bytes = 67072 * N
    row_bytes, call_steps, call_ms = N * d * 2, 64, 0.0
    for c in range(steps // call_steps):
        sl = slice(c * call_steps, (c + 1) * call_steps)
        qs[sl].mul_(1.0); ks[sl].mul_(1.0); vs[sl].mul_(1.0)
        call_ms += _event_time_ms(torch, lambda: run_decode(call_steps, c * call_steps * row_bytes), 1)
    ex["decode"] = {"workload": "configs[3]: batch 64 x 16 heads, head_dim 64, proj_dim 64, 2048 steps after a "
                                "512-token prefill, fused feature map, fp32 state in place, one launch per step; the "
                                "q, k, v rows of a step are written on the device just before it (64-step calls)",
                    "tokens_per_s": round(B * steps / (call_ms * 1e-3), 1), "us_per_step": round(1e3 * call_ms / steps, 3),
                    "algorithmic_bytes_per_step": step_bytes,
                    "hbm_gbs": round(step_bytes * steps / (call_ms * 1e-3) / 1e9, 1),
                    "hbm_frac": round(step_bytes * steps / (call_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                    "note": "the 33.5 MB state fits the 256 MB last-level cache, which serves most of its reads; "
                            "profiles/ holds the FETCH_SIZE / WRITE_SIZE bytes per step"}
    # (2) the same 2048 steps as one C call over pre-generated rows (the library streams the rows of
    # coming steps through a touch kernel first: rows that a decoder would not have yet)
    s.copy_(s0); z.copy_(z0)
    ms = _event_time_ms(torch, lambda: run_decode(steps), 1)
    ex["decode"]["one_call_pregenerated_rows"] = {
        "us_per_step": round(1e3 * ms / steps, 3),
        "hbm_frac": round(step_bytes * steps / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    # parity of the first steps against the oracle on 2 heads
    s.copy_(s0); z.copy_(z0)
    _lib.check(lib.rfa_incremental_fused(p(qs), p(ks), p(vs), p(W), O.SCALE, p(s), p(z), p(outs), 8, B, H, D, d, stream))
    torch.cuda.synchronize()
    Wc = W.float().cpu()[:2]
    fq = O.random_project(qs[:8, :1, :2].float().cpu(), Wc).reshape(8, 2, K)
    fk = O.random_project(ks[:8, :1, :2].float().cpu(), Wc).reshape(8, 2, K)
    want, _, _ = O.causal_forward_loop(fq, fk, vs[:8, :1, :2].float().cpu().reshape(8, 2, d),
                                       s0[:1, :2].cpu().reshape(2, K, d), z0[:1, :2].cpu().reshape(2, K))
    ex["decode"]["parity_max_abs"] = (outs[:8, :1, :2].float().cpu().reshape(8, 2, d) - want).abs().max().item()
    dec_gbs = ex["decode"]["hbm_gbs"]
    ex["decode"]["roofline"] = {"bound": "hbm", "kernel": "k_decode_step", "achieved": dec_gbs, "peak": HBM_PEAK_GBS,
                                "unit": "GB/s", "frac": round(dec_gbs / HBM_PEAK_GBS, 4),
                                "traffic": _profile_traffic_bytes("k_decode_step<128, 64, true>"),
                                "traffic_source": TRAFFIC_PROFILE, "bytes_per_launch": step_bytes}
    if "cpu" not in skip:
        # the reference's decode loop (causal_attention.py:42-50) with its feature map, fp32 torch-CPU, whole batch,
        # from the same prefilled state, on the first rows of the run
        cores = _cpu_threads(torch)
        n_cpu = 48
        Wf = W.float().cpu()
        cq_, ck_, cv_ = (t[:n_cpu].float().cpu() for t in (qs, ks, vs))
        cs_, cz_ = s0.cpu().reshape(N, K, d).clone(), z0.cpu().reshape(N, K).clone()

        def cpu_decode(steps_):
            s_, z_ = cs_, cz_
            for t in range(steps_):
                fq_ = O.random_project(cq_[t:t + 1], Wf).reshape(N, K)
                fk_ = O.random_project(ck_[t:t + 1], Wf).reshape(N, K)
                _, s_, z_ = O.incremental_step(fq_, fk_, cv_[t].reshape(N, d), s_, z_)
        cpu_decode(4)
        t0 = time.perf_counter()
        cpu_decode(n_cpu)
        tcpu = (time.perf_counter() - t0) / n_cpu
        ex["decode"]["cpu_baseline"] = {
            "value": round(B / tcpu, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{n_cpu} of the {steps} steps (the first ones, whole batch of {B} x {H} heads) after 4 warm-up steps: "
                      "feature maps of q, k and the loop-form step (causal_attention.py:42-50) in fp32 torch-CPU",
            "us_per_step": round(1e6 * tcpu, 1), "speedup": round(ex["decode"]["tokens_per_s"] / (B / tcpu), 1)}
    del qs, ks, vs, outs
    if "decode_module" not in skip:
        # (3) through the API the reference exposes: one CausalAttention.forward(x[1], W, saved_state=state)
        # per token (causal_attention.py:249-265), q/k/v/out projections included; eager calls, then the
        # same step captured once into a HIP graph (state advanced in place) and replayed
        from rfa_amd import CausalAttention
        torch.manual_seed(0)
        E = H * d
        dec = CausalAttention(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).to(dev).half().eval()
        xs = (torch.randn(256, B, E, generator=g) * 0.5).half().to(dev)
        shape4 = (B, H, K, d)
        with torch.no_grad():
            state = {"prev_s": s0.view(shape4).clone(), "prev_z": z0.view(B, H, K).clone()}
            y_first = dec(xs[0:1], W, saved_state=state).clone()
            for t in range(1, 16):
                dec(xs[t:t + 1], W, saved_state=state)
            torch.cuda.synchronize()
            _lib.check(lib.rfa_profile_reset()); _lib.check(lib.rfa_profile_enable(1))
            t0 = time.perf_counter()
            for t in range(steps):
                dec(xs[t % 256:t % 256 + 1], W, saved_state=state)
            torch.cuda.synchronize()
            eager_s = time.perf_counter() - t0
            _lib.check(lib.rfa_profile_enable(0))
            step_kernel_us = {n_: round(1e3 * ms_ / c_, 2) for n_, (ms_, c_) in _lib.profile_totals().items()}
            dec.decode_inplace = True
            gstate = {"prev_s": s0.view(shape4).clone(), "prev_z": z0.view(B, H, K).clone()}
            gs, gz = gstate["prev_s"], gstate["prev_z"]
            xg = xs[0:1].clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    dec(xg, W, saved_state=gstate)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                yg = dec(xg, W, saved_state=gstate)
            in_place = gstate["prev_s"] is gs and gstate["prev_z"] is gz
            gs.copy_(s0.view(shape4)); gz.copy_(z0.view(B, H, K))
            graph.replay()
            torch.cuda.synchronize()
            graph_ok = bool(in_place and torch.equal(yg, y_first))
            for _ in range(16):
                graph.replay()
            graph_ms = _event_time_ms(torch, graph.replay, steps)
        ex["decode"]["module_per_token"] = {
            "workload": "CausalAttention(embed 1024, 16 heads).forward(x[1, 64, 1024], W, saved_state) per token, 2048 tokens",
            "eager_us_per_step": round(1e6 * eager_s / steps, 2), "eager_tokens_per_s": round(B * steps / eager_s, 1),
            "hip_graph_replay_us_per_step": round(1e3 * graph_ms, 2),
            "hip_graph_tokens_per_s": round(B / (graph_ms * 1e-3), 1),
            "decode_kernel_us": step_kernel_us.get("k_decode_step"), "library_kernels_us": step_kernel_us,
            "graph_equals_eager": graph_ok}
        del dec, graph, xs, state, gstate

    # ---- cross attention (config 3): T256 S512 B32 H8, lengths U[256, 512]
    Tt, S, B, H = 256, 512, 32, 8
    N = B * H
    g = torch.Generator(device="cpu").manual_seed(1234 + 3)
    W = O.make_w(d, D, H).half().to(dev)
    lens = torch.randint(256, 513, (B,), generator=g)
    pad = (torch.arange(S)[None, :] >= lens[:, None]).to(torch.uint8).to(dev)
    pk = rfa_hip.feature_map_forward(unit(torch.randn(S, B, H, d, generator=g)).half().to(dev), W, O.SCALE)
    pq = rfa_hip.feature_map_forward(unit(torch.randn(Tt, B, H, d, generator=g)).half().to(dev), W, O.SCALE)
    v = torch.randn(S, B, H, d, generator=g).half().to(dev)
    go = torch.randn(Tt, B, H, d, generator=g).half().to(dev)

    def cross_step():
        s_, z_ = rfa_hip.cross_state(pk, v, pad)
        rfa_hip.cross_readout(pq, s_, z_)
        _, ds, dz = rfa_hip.cross_readout_backward(pq, s_, z_, go)
        rfa_hip.cross_state_backward(pk, v, ds, dz, pad)
    for _ in range(5):
        cross_step()
    ms = _event_time_ms(torch, cross_step, 50)
    flops = 6 * K * d * float((lens + Tt).sum()) * H
    # algorithmic bytes of one forward + backward at the feature-level boundary, every tensor at its
    # full shape, read or written once by each of the four steps that needs it:
    #   state           reads phi_k, v [S]                      writes s, z
    #   readout         reads phi_q [T], s, z                   writes attn [T]
    #   readout backward reads phi_q, grad [T], s, z            writes dphi_q [T], ds, dz
    #   state backward  reads phi_k, v [S], ds, dz              writes dphi_k, dv [S]
    st_bytes = (K * d + K) * 4
    per_seq = (S * (K + d) * 2 + st_bytes) + (Tt * K * 2 + st_bytes + Tt * d * 2) \
        + (Tt * (K + d) * 2 + st_bytes + Tt * K * 2 + st_bytes) + (S * (K + d) * 2 + st_bytes + S * (K + d) * 2)
    cross_bytes = per_seq * N
    _lib.check(lib.rfa_profile_reset()); _lib.check(lib.rfa_profile_enable(1))
    for _ in range(20):
        cross_step()
    torch.cuda.synchronize()
    _lib.check(lib.rfa_profile_enable(0))
    cross_kernels = {n_: round(1e3 * ms_ / c_, 2) for n_, (ms_, c_) in _lib.profile_totals().items()}
    ex["cross"] = {"workload": "configs[2]: tgt 256, src 512, batch 32, 8 heads, lengths U[256,512], fwd+bwd",
                   "tgt_tokens_per_s": round(B * Tt / (ms * 1e-3), 1), "us_per_step": round(1e3 * ms, 2),
                   "algorithmic_tflops": round(flops / (ms * 1e-3) / 1e12, 2),
                   "kernels_us": cross_kernels,
                   "roofline": {"bound": "hbm", "achieved": round(cross_bytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                                "unit": "GB/s", "frac": round(cross_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                "algorithmic_bytes": cross_bytes,
                                "mfma_frac_of_2500_tflops": round(flops / (ms * 1e-3) / 1e12 / 2500.0, 4)}}

    if "cpu" not in skip:
        # the reference's einsum formulas (cross_attention.py:97-104, 266-269) and their closed-form gradients in fp32
        # torch-CPU on the whole configuration
        cores = _cpu_threads(torch)
        cpk, cpq, cv_, cgo = (t.float().cpu() for t in (pk, pq, v, go))
        cmask = pad.bool().cpu().t().contiguous()        # [S, B], True = pad

        def cpu_cross():
            s_, z_ = O.cross_state(cpk, cv_, cmask)
            O.cross_readout(cpq, s_, z_)
            _, ds_, dz_ = O.cross_readout_backward(cpq, s_, z_, cgo)
            O.cross_state_backward(cpk, cv_, ds_, dz_, cmask)
        cpu_cross()
        ctimes = []
        for _ in range(3):
            t0 = time.perf_counter()
            cpu_cross()
            ctimes.append(time.perf_counter() - t0)
        tcpu = min(ctimes)
        ex["cross"]["cpu_baseline"] = {
            "value": round(B * Tt / tcpu, 1), "unit": "tgt tokens/s", "cores": cores, "kind": "port",
            "sample": "the whole configuration (32 x 8 sequences), state + readout + both backward formulas in fp32 "
                      "torch-CPU, 1 warm-up, best of 3",
            "ms_per_step": round(1e3 * tcpu, 2), "speedup": round(ex["cross"]["tgt_tokens_per_s"] / (B * Tt / tcpu), 1)}
    ex["cross"]["roofline"]["traffic"] = _profile_traffic_bytes(
        "k_segment_state<128, 64, 4, false, true>", "k_causal_fwd<128, 64, 4, false>", "k_causal_bwd_dq<128, 64, 8, false>",
        "k_causal_bwd_dkdv<128, 64, 4, false, false>")
    ex["cross"]["roofline"]["traffic_source"] = TRAFFIC_PROFILE + " (sum of the four kernels)"

    # ---- long-context causal fwd+bwd (config 5): seq 16384, batch 2, 16 heads, head_dim 128, proj_dim 128
    T5, B5, H5, d5, D5 = 16384, 2, 16, 128, 128
    N5, K5 = B5 * H5, 2 * D5
    W5 = O.make_w(d5, D5, H5).half().to(dev)
    g5 = torch.Generator(device="cpu").manual_seed(1234 + 5)
    mk = lambda last: torch.randn(T5, B5, H5, last, generator=g5)
    pq5 = rfa_hip.feature_map_forward(unit(mk(d5)).half().to(dev), W5, O.SCALE).view(T5, N5, K5)
    pk5 = rfa_hip.feature_map_forward(unit(mk(d5)).half().to(dev), W5, O.SCALE).view(T5, N5, K5)
    v5 = mk(d5).half().to(dev).view(T5, N5, d5)
    go5 = mk(d5).half().to(dev).view(T5, N5, d5)

    o5 = torch.empty_like(v5)
    dq5, dk5, dv5 = torch.empty_like(pq5), torch.empty_like(pk5), torch.empty_like(v5)
    fb5 = lib.rfa_causal_forward_workspace_bytes(T5, N5, K5, d5)
    bb5 = lib.rfa_causal_backward_workspace_bytes(T5, N5, K5, d5)
    sb5 = lib.rfa_causal_saved_state_bytes(T5, N5, K5, d5)
    ws5 = torch.empty(max(fb5, bb5, 1), dtype=torch.uint8, device=dev)
    sv5 = torch.empty(max(sb5, 1), dtype=torch.uint8, device=dev)

    def long_step():
        _lib.check(lib.rfa_causal_forward_save(p(pq5), p(pk5), p(v5), p(o5), p(sv5), sb5, T5, N5, K5, d5,
                                               p(ws5), fb5, stream))
        _lib.check(lib.rfa_causal_backward_saved(p(pq5), p(pk5), p(v5), p(go5), p(o5), p(sv5), sb5, p(dq5), p(dk5),
                                                 p(dv5), T5, N5, K5, d5, p(ws5), bb5, stream))
    for _ in range(10):                                     # the oracle work above left the GPU idle: let the clocks settle
        long_step()
    ms = _event_time_ms(torch, long_step, 20)
    ns = 2                                                  # parity on two sequences (chunked-exact oracle)
    sl = lambda t: t[:, :ns].float().cpu()
    cores = _cpu_threads(torch)
    c5 = [sl(t) for t in (pq5, pk5, v5, go5)]
    t0 = time.perf_counter()
    ref5 = O.causal_forward_chunked(*c5[:3])
    rq5, rk5, rv5 = O.causal_backward_chunked(*c5)
    tcpu5 = time.perf_counter() - t0
    rel = lambda a, b: ((a - b).norm() / b.norm()).item()
    bytes5 = (2 * K5 * 2 + 2 * d5 * 2 + 2 * K5 * 2 + 2 * d5 * 2 + 2 * K5 * 2 + d5 * 2) * N5 * T5   # 4352 B per (head, token)
    ex["long_context"] = {"workload": "configs[4]: seq 16384, batch 2, 16 heads, head_dim 128, proj_dim 128 (phi width 256), "
                                      "causal fwd+bwd (saved pair)",
                          "tokens_per_s": round(B5 * T5 / (ms * 1e-3), 1), "ms_per_step": round(ms, 4),
                          "algorithmic_bytes": bytes5, "frac_of_hbm": round(bytes5 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                          "parity": {"out_max_abs": (sl(o5) - ref5).abs().max().item(), "dq_rel": rel(sl(dq5), rq5),
                                     "dk_rel": rel(sl(dk5), rk5), "dv_rel": rel(sl(dv5), rv5)}}
    gbs5 = bytes5 / (ms * 1e-3) / 1e9
    ex["long_context"]["roofline"] = {
        "bound": "hbm", "achieved": round(gbs5, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs5 / HBM_PEAK_GBS, 4),
        "traffic": _profile_traffic_bytes("k_segment_state<256, 128, 8, true, false>", "k_totals_scan<false>",
                                          "k_causal_fwd<256, 128, 8, true>", "k_causal_bwd_dq_saved<128, 128, 8, 8, 256>",
                                          "k_totals_scan<true>", "k_causal_bwd_dkdv_roles<256, 128, 8>"),
        "traffic_source": TRAFFIC_PROFILE + " (sum of the step's kernels)", "bytes_per_step": bytes5}
    ex["long_context"]["cpu_baseline"] = {
        "value": round(ns * T5 / H5 / tcpu5, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"{ns} of the {N5} sequences (T={T5}), forward + backward in the oracle's chunked form (the cumulative-sum "
                  "form would need 64 GiB) in fp32 torch-CPU, one run (the parity check of this section)",
        "seconds": round(tcpu5, 2), "speedup": round(ex["long_context"]["tokens_per_s"] / (ns * T5 / H5 / tcpu5), 1)}
    del pq5, pk5, v5, go5, o5, dq5, dk5, dv5, ws5, sv5

    # ---- feature map (config 2 shape): phi forward + backward for q
    T, B, H = 1024, 8, 8
    x = torch.randn(T, B, H, d, generator=g).half().to(dev)
    gp = torch.randn(T, B, H, 2 * D, generator=g).half().to(dev)
    R = T * B
    phi, dx = torch.empty_like(gp), torch.empty_like(x)
    dw = torch.empty(H, D, d, dtype=torch.float32, device=dev)
    wbytes = lib.rfa_feature_map_backward_workspace_bytes(R, H, D, d)
    fws = torch.empty(max(wbytes, 1), dtype=torch.uint8, device=dev)
    f = lambda: _lib.check(lib.rfa_feature_map_forward(p(x), p(W), p(phi), R, H, D, d, O.SCALE, stream))
    b = lambda: _lib.check(lib.rfa_feature_map_backward(p(x), p(W), p(gp), p(dx), p(dw), R, H, D, d, O.SCALE,
                                                        p(fws), wbytes, stream))
    for _ in range(5):
        f(); b()
    tf, tb = _event_time_ms(torch, f, 100), _event_time_ms(torch, b, 100)
    x_b, phi_b = torch.randn(T, B, H, d, generator=g).half().to(dev), torch.empty_like(gp)
    fp_ = lambda: _lib.check(lib.rfa_feature_map_forward_pair(p(x), p(x_b), p(W), p(phi), p(phi_b), R, H, D, d, O.SCALE, stream))
    for _ in range(5):
        fp_()
    tfp = _event_time_ms(torch, fp_, 100)
    rows = R * H
    ex["feature_map"] = {"workload": "phi of [1024, 8, 8, 64] -> [.., 128]; back-to-back launches through the C ABI",
                         "fwd_us": round(1e3 * tf, 2), "bwd_us": round(1e3 * tb, 2), "fwd_pair_us": round(1e3 * tfp, 2),
                         "fwd_hbm_gbs": round(rows * (d + 2 * D) * 2 / (tf * 1e-3) / 1e9, 1),
                         "bwd_hbm_gbs": round(rows * (2 * d + 2 * D) * 2 / (tb * 1e-3) / 1e9, 1)}
    # ---- raw boundary (config 2): q, k, v [T, B, H, d] in, dq, dk, dv out -- the feature maps of q
    # and k, the causal forward and backward, and the feature-map backward pair, through the C ABI
    # (1408 algorithmic bytes per (head, token): 3 + 1 + 4 + 3 rows of d halves)
    q2 = unit(torch.randn(T, B, H, d, generator=g)).half().to(dev)
    k2 = unit(torch.randn(T, B, H, d, generator=g)).half().to(dev)
    v2 = torch.randn(T, B, H, d, generator=g).half().to(dev)
    g2 = torch.randn(T, B, H, d, generator=g).half().to(dev)
    N2, K2 = B * H, 2 * D
    pq2, pk2 = torch.empty(T, N2, K2, dtype=torch.float16, device=dev), torch.empty(T, N2, K2, dtype=torch.float16, device=dev)
    o2 = torch.empty(T, N2, d, dtype=torch.float16, device=dev)
    dpq, dpk, dv2 = torch.empty_like(pq2), torch.empty_like(pk2), torch.empty_like(o2)
    dq2, dk2 = torch.empty_like(q2), torch.empty_like(k2)
    fb2 = lib.rfa_causal_forward_workspace_bytes(T, N2, K2, d)
    bb2 = lib.rfa_causal_backward_workspace_bytes(T, N2, K2, d)
    sb2 = lib.rfa_causal_saved_state_bytes(T, N2, K2, d)
    pb2 = lib.rfa_feature_map_backward_pair_workspace_bytes(R, H, D, d)
    ws2 = torch.empty(max(fb2, bb2, pb2, 1), dtype=torch.uint8, device=dev)
    sv2 = torch.empty(max(sb2, 1), dtype=torch.uint8, device=dev)

    def raw_step():
        _lib.check(lib.rfa_feature_map_forward_pair(p(q2), p(k2), p(W), p(pq2), p(pk2), R, H, D, d, O.SCALE, stream))
        _lib.check(lib.rfa_causal_forward_save(p(pq2), p(pk2), p(v2), p(o2), p(sv2), sb2, T, N2, K2, d, p(ws2), fb2, stream))
        _lib.check(lib.rfa_causal_backward_saved(p(pq2), p(pk2), p(v2), p(g2), p(o2), p(sv2), sb2, p(dpq), p(dpk), p(dv2),
                                                 T, N2, K2, d, p(ws2), bb2, stream))
        _lib.check(lib.rfa_feature_map_backward_pair(p(q2), p(k2), p(W), p(dpq), p(dpk), p(dq2), p(dk2), p(dw), R, H, D, d,
                                                     O.SCALE, p(ws2), pb2, stream))
    for _ in range(5):
        raw_step()
    traw = _event_time_ms(torch, raw_step, 100)
    raw_bytes = 22 * d * N2 * T
    ex["raw_boundary"] = {"workload": "configs[1] from raw q, k, v to dq, dk, dv: phi(q) and phi(k) in one launch, causal "
                                      "fwd+bwd, phi backward pair",
                          "us_per_step": round(1e3 * traw, 2), "tokens_per_s": round(B * T / (traw * 1e-3), 1),
                          "algorithmic_bytes": raw_bytes,
                          "frac_of_hbm": round(raw_bytes / (traw * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    del q2, k2, v2, g2, pq2, pk2, o2, dpq, dpk, dv2, dq2, dk2, ws2, sv2

    # ---- whole CausalAttention module (config 2 shape, embed 512): forward + backward of the module
    # with its projections on the library's kernels, the same module on nn.Linear + separate phi
    # launches, and the fused module replayed from a HIP graph (no host work per step)
    from rfa_amd import CausalAttention
    torch.manual_seed(0)
    E = H * d
    mod = CausalAttention(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).to(dev).half()
    mx = (torch.randn(T, B, E, generator=g) * 0.5).half().to(dev).requires_grad_(True)
    mg = torch.randn(T, B, E, generator=g).half().to(dev)

    def mstep():
        mod.zero_grad(set_to_none=True)
        mx.grad = None
        y = mod(mx, W)
        y.backward(mg)
        return y

    def timed(fn, n=20):
        for _ in range(3):
            fn()
        return 1e3 * _event_time_ms(torch, fn, n)

    fused_us = timed(mstep)
    mod.fuse_projections = False
    unfused_us = timed(mstep)
    mod.fuse_projections = True
    y_eager = mstep().detach().clone()
    gx_eager = mx.grad.detach().clone()
    import warnings
    # the warm-up below runs the step on a side stream on purpose (graph capture needs one)
    warnings.filterwarnings("ignore", message="The AccumulateGrad node's stream does not match")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            mstep()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    mod.zero_grad(set_to_none=True)
    mx.grad = None
    with torch.cuda.graph(graph):
        y_graph = mod(mx, W)
        y_graph.backward(mg)
    graph_us = timed(graph.replay)
    mstep()                                      # eager work between replays
    graph.replay()
    torch.cuda.synchronize()
    ex["module_step"] = {"workload": "CausalAttention(embed 512, 8 heads) forward + backward on [1024, 8, 512] fp16",
                         "eager_us": round(fused_us, 1), "eager_library_projections_us": round(unfused_us, 1),
                         "hip_graph_replay_us": round(graph_us, 1),
                         "graph_equals_eager": bool(torch.equal(y_graph, y_eager) and torch.equal(mx.grad, gx_eager))}
    del graph, mod

    # ---- matrix-pipe rate of the MFMA instruction the kernels use (register operands, no memory
    # traffic): the fp16 figure this device delivers, next to the published 2.5 PFLOP/s
    import ctypes
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    flops = ctypes.c_double(0.0)
    rates = {}
    for wps in (1, 2, 4):
        probe = lambda: _lib.check(lib.rfa_selftest_mfma_rate(wps, 4096, p(sink), ctypes.byref(flops), stream))
        for _ in range(3):
            probe()
        tp = _event_time_ms(torch, probe, 10)
        rates[f"waves_per_simd_{wps}"] = round(flops.value / (tp * 1e-3) / 1e12, 1)
    ex["mfma_rate"] = {"instruction": "v_mfma_f32_16x16x32_f16, 8 independent accumulators per wave",
                       "tflops": rates, "published_dense_fp16_tflops": 2500.0}

    # ---- plain device copy of 512 MiB (larger than the 256 MiB last-level cache): the HBM
    # bandwidth a trivial kernel reaches here, and the known-size dispatch against which the
    # rocprofv3 FETCH_SIZE / WRITE_SIZE counters are scaled
    src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    cp = lambda: torch.bitwise_not(src, out=dst)      # an elementwise kernel, not a DMA copy
    for _ in range(2):
        cp()
    tc = _event_time_ms(torch, cp, 5)
    ex["hbm_copy"] = {"bytes_read": 512 << 20, "bytes_written": 512 << 20,
                      "gbs": round(2 * (512 << 20) / (tc * 1e-3) / 1e9, 1)}
    return ex


if __name__ == "__main__":
    main()
