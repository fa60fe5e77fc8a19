#!/usr/bin/env python3
"""Benchmark of the MoE layer (router -> dispatch -> MXFP4 expert MLP -> combine)
on one MI355X through the C ABI.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tokens T]

Prints ONE JSON line.  A step is one forward of the layer over one batch of T
synthetic tokens with weights, input and output resident in HBM.  `value` is
tokens/s of the whole layer; `roofline` describes the dominant kernel (gate/up
projections), timed live with HIP events on the library's stream;
`cpu_baseline` is the CPU checker (a restatement of the reference's
single-threaded path) timed on this host on a bounded sample.

Workloads (BASELINE.json configs):
  c2_20b_decode   32 experts, top-4, H = F = 2880, T in {1,2,4,8,16,32,64} (default, T=16)
  c3_20b_prefill  same layer, T = 2048
  c4_120b         128 experts, 8 hot experts (+2.0 router bias), T in {1,16,4096}
  c5_stack        36 layers of the 120b shape with RMSNorm + residual, T in {1,8,64}
Neighbouring paths (not the headline):
  gguf_ingest     one 20b-shaped block from a GGUF file into a resident layer
  f16_20b_decode  the 20b-shaped layer with fp16 experts (the reference's other expert branch), T = 16
  f16_20b_prefill same, T = 2048
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP4_PEAK_TFLOPS = 10100.0  # dense MXFP4, published
MFMA_F16_PEAK_TFLOPS = 2500.0   # dense fp16, published

SHAPES = {
    "c2_20b_decode": dict(E=32, k=4, H=2880, F=2880, hot=0, default_T=16, sweep=[1, 2, 4, 8, 16, 32, 64]),
    "c3_20b_prefill": dict(E=32, k=4, H=2880, F=2880, hot=0, default_T=2048, sweep=[]),
    "c4_120b": dict(E=128, k=4, H=2880, F=2880, hot=8, default_T=16, sweep=[1, 16]),
    "c5_stack": dict(E=128, k=4, H=2880, F=2880, hot=8, default_T=8, sweep=[1, 8, 64], layers=36),
    # next-row workload: one 20b-shaped block read from a GGUF file into a resident layer
    "gguf_ingest": dict(E=32, k=4, H=2880, F=2880, hot=0, default_T=4, sweep=[]),
    # next-row workloads: the same layer with fp16 experts
    "f16_20b_decode": dict(E=32, k=4, H=2880, F=2880, hot=0, default_T=16, sweep=[1, 4, 16, 64], f16=True),
    "f16_20b_prefill": dict(E=32, k=4, H=2880, F=2880, hot=0, default_T=2048, sweep=[], f16=True),
}


def matrix_bytes(rows, K, f16=False):
    """One expert matrix: fp16, or MXFP4 in 17-byte blocks of 32."""
    return rows * K * 2 if f16 else rows * (K // 32) * 17


def layer_bytes(E, k, H, F, T, U, f16=False):
    """Algorithmic HBM bytes of one layer forward: every distinct expert's three
    matrices and biases once, the router weights, activations in and out, router
    output."""
    mat_gu = matrix_bytes(F, H, f16)
    mat_d = matrix_bytes(H, F, f16)
    return U * (2 * mat_gu + mat_d + (2 * F + H) * 4) + E * H * 4 + E * 4 + 2 * T * H * 4 + T * k * 8


def gateup_bytes(H, F, T, k, U, f16=False):
    """Algorithmic bytes of the gate/up kernel: both matrices and biases of every
    distinct expert once, the fp32 activations in, the fp32 activations out."""
    return U * (2 * matrix_bytes(F, H, f16) + 2 * F * 4) + T * H * 4 + T * k * F * 4


def layer_flops(E, k, H, F, T):
    return T * (k * 6 * H * F + 2 * E * H)


def make_layer(lib, synth, shape, seed, layer_index=0, norm=False):
    L = synth.LayerInputs(shape["E"], shape["k"], shape["H"], shape["F"], seed=seed, layer=layer_index,
                          hot_experts=shape["hot"], with_norm=norm)
    f16 = bool(shape.get("f16"))
    layer = lib.layer(L.E, L.k, L.H, L.F, f16=f16)
    layer.set_router(L.gate_w, L.gate_b)
    layer.fill_synthetic(L.seed, L.layer)
    for e in range(L.E):
        if f16:
            layer.set_expert_f16(e, None, None, None, L.b_up[e], L.b_gate[e], L.b_down[e])
        else:
            layer.set_expert(e, None, None, None, L.b_up[e], L.b_gate[e], L.b_down[e])
    if norm:
        layer.set_norm(L.norm_w, 1e-5)
    return L, layer


def bench_gguf_ingest(lib, synth, shape, reps=3):
    """Writes a synthetic one-block GGUF file (MXFP4 experts, biases, router, norm) and
    times csk_layer_from_gguf: file -> host -> HBM -> repacked resident planes."""
    import tempfile
    from coalsack_amd import gguf_writer as gw
    L = synth.LayerInputs(shape["E"], shape["k"], shape["H"], shape["F"], seed=7, with_norm=True)
    meta = [("general.architecture", gw.STR, "gpt-oss"), ("gpt-oss.expert_count", gw.U32, L.E),
            ("gpt-oss.expert_used_count", gw.U32, L.k)]
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "block.gguf")
        gw.write_gguf(path, meta, gw.moe_block_tensors(L, 0))
        nbytes = os.path.getsize(path)
        times = []
        with lib.gguf(path) as g:
            for _ in range(reps):
                t0 = time.perf_counter()
                layer = g.layer(0)
                lib.synchronize()
                times.append(time.perf_counter() - t0)
                hidden = synth.hidden_states(4, L.H, seed=1)
                out = layer.forward(hidden)
                ok = bool(np.array_equal(layer.export(L.E - 1, 2), L.blocks(L.E - 1, 2)))
                layer.close()
    return dict(file_bytes=nbytes, seconds=min(times), all_seconds=times, roundtrip_ok=ok,
                finite=bool(np.all(np.isfinite(out))))


def time_forward(lib, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    lib.synchronize()
    e0, e1 = lib.event(), lib.event()
    lib.record(e0)
    for _ in range(steps):
        fn()
    lib.record(e1)
    ms = lib.elapsed_ms(e0, e1)
    lib.synchronize()
    lib.dll.csk_event_destroy(e0)
    lib.dll.csk_event_destroy(e1)
    return ms / steps


def stage_profile(lib, fn, steps):
    lib.stage_timing(True)
    acc = {}
    for _ in range(steps):
        fn()
        for kk, v in lib.stage_times().items():
            acc[kk] = acc.get(kk, 0.0) + v
    lib.stage_timing(False)
    return {kk: v / steps for kk, v in acc.items()}


def close_calls(L, hidden, k):
    """Tokens whose k+1 largest router logits contain two closer than the library's
    close-call threshold (8 * 2^-24 * sqrt(H), relative to max(1, |logit|)): those are
    recomputed in the reference's summation order, which costs tens of microseconds."""
    lg = hidden.astype(np.float64) @ L.gate_w.astype(np.float64).T + L.gate_b
    srt = -np.sort(-lg, axis=1)[:, :k + 1]
    gaps = (srt[:, :-1] - srt[:, 1:]) / np.maximum(1.0, np.abs(srt[:, :-1]))
    return int(np.count_nonzero(gaps.min(axis=1) <= 8 * 5.96e-8 * np.sqrt(hidden.shape[1])))


def bench_layer(lib, synth, shape, T, steps, warmup, seed=1234):
    """Times the forward over `nb` different token batches in rotation (decode sizes: the
    set of selected experts, and with it the bytes streamed, varies from batch to batch)."""
    L, layer = make_layer(lib, synth, shape, seed)
    nb = 8 if T < 512 else 1
    hiddens = [synth.hidden_states(T, L.H, seed=T + 1000 * i) for i in range(nb)]
    d_ins = [lib.to_device(h) for h in hiddens]
    d_out = lib.dev_alloc(hiddens[0].nbytes)
    turn = [0]

    def fn():
        layer.forward_device(d_ins[turn[0] % nb], T, d_out)
        turn[0] += 1
    steps = (steps + nb - 1) // nb * nb
    ms = time_forward(lib, fn, steps, (warmup + nb - 1) // nb * nb)
    stages = stage_profile(lib, fn, (max(5, min(steps, 50)) + nb - 1) // nb * nb)
    Us, tmax = [], 0
    for i in range(nb - 1, -1, -1):  # batch 0 last: its output is the one checked
        layer.forward_device(d_ins[i], T, d_out)
        if T <= 32768:
            counts, _ = layer.last_dispatch(T)
            Us.append(int(np.count_nonzero(counts)))
            tmax = max(tmax, int(counts.max()))
        else:  # taken in several passes: no single dispatch to read back; every expert is in use
            Us.append(shape["E"])
    U = float(np.mean(Us))
    hidden = hiddens[0]
    out = lib.to_host(d_out, (T, L.H))
    f16 = bool(shape.get("f16"))
    L.f16_weights = None
    if f16:
        # the CPU leg needs the generated halves of the experts its token sample selects
        from coalsack_amd import capi
        ns = min(T, 2)
        _, pairs = layer.forward(hidden[:ns], want_pairs=True)
        L.f16_weights = {int(e): [layer.export_f16(int(e), w) for w in (capi.W_UP, capi.W_GATE, capi.W_DOWN)]
                         for e in sorted(set(pairs[..., 0].astype(int).ravel().tolist()))}
        L.f16_sample = ns
    for d in d_ins:
        lib.dev_free(d)
    lib.dev_free(d_out)
    layer.close()
    res = dict(T=T, ms_per_step=ms, tokens_per_s=T / (ms * 1e-3), distinct_experts=U,
               stage_ms=stages, finite=bool(np.all(np.isfinite(out))),
               max_tokens_per_expert=tmax, batches=nb, steps=steps,
               close_call_tokens=sum(close_calls(L, h, L.k) for h in hiddens))
    res["layer_bytes"] = layer_bytes(L.E, L.k, L.H, L.F, T, U, f16)
    res["layer_hbm_frac"] = res["layer_bytes"] / (ms * 1e-3) / (HBM_PEAK_GBS * 1e9)
    res["layer_flops"] = layer_flops(L.E, L.k, L.H, L.F, T)
    res["layer_fp4_frac"] = res["layer_flops"] / (ms * 1e-3) / (MFMA_FP4_PEAK_TFLOPS * 1e12)
    gu = gateup_bytes(L.H, L.F, T, L.k, U, f16)
    res["gateup_bytes"] = gu
    res["gateup_gbs"] = gu / (stages["gateup"] * 1e-3) / 1e9
    return res, (L, hidden, out)


def bench_stack(lib, synth, shape, T, steps, warmup, n_layers, seed=1234):
    layers = []
    for i in range(n_layers):
        _, layer = make_layer(lib, synth, shape, seed, layer_index=i, norm=True)
        layers.append(layer)
    from coalsack_amd.capi import stack_forward
    hidden = synth.hidden_states(T, shape["H"], seed=T)
    d_h = lib.to_device(hidden)
    d_h0 = lib.to_device(hidden)

    def fn():
        # the stack updates the hidden states in place; start every step from the same N(0,1) input
        lib.copy_d2d(d_h, d_h0, hidden.nbytes)
        stack_forward(lib, layers, d_h, T)
    ms = time_forward(lib, fn, steps, warmup)
    out = lib.to_host(d_h, hidden.shape)
    # untimed pass, layer by layer, to count the distinct experts each layer streams
    from coalsack_amd.capi import FWD_RMSNORM, FWD_RESIDUAL
    lib.copy_d2d(d_h, d_h0, hidden.nbytes)
    total_bytes, distinct = 0, []
    for layer in layers:
        layer.forward_device(d_h, T, d_h, FWD_RMSNORM | FWD_RESIDUAL)
        counts, _ = layer.last_dispatch(T)
        U = int(np.count_nonzero(counts))
        distinct.append(U)
        total_bytes += layer_bytes(shape["E"], shape["k"], shape["H"], shape["F"], T, U) + shape["H"] * 4
    lib.dev_free(d_h)
    lib.dev_free(d_h0)
    for layer in layers:
        layer.close()
    return dict(T=T, layers=n_layers, ms_per_step=ms, tokens_per_s=T / (ms * 1e-3),
                finite=bool(np.all(np.isfinite(out))), stack_bytes=total_bytes,
                distinct_experts_per_layer=distinct)


def measured_copy_gbs(lib, nbytes=256 << 20, reps=10):
    """What a plain copy kernel reaches on this box (bytes read + bytes written per second):
    the practical ceiling beside the 8 TB/s on the data sheet."""
    src, dst = lib.dev_alloc(nbytes), lib.dev_alloc(nbytes)
    lib.copy_d2d(dst, src, nbytes)  # first touch
    e0, e1 = lib.event(), lib.event()
    lib.record(e0)
    for _ in range(reps):
        lib.copy_d2d(dst, src, nbytes)
    lib.record(e1)
    lib.synchronize()
    ms = lib.elapsed_ms(e0, e1)
    lib.dll.csk_event_destroy(e0)
    lib.dll.csk_event_destroy(e1)
    lib.dev_free(src)
    lib.dev_free(dst)
    return 2 * nbytes * reps / (ms * 1e-3) / 1e9


def cpu_baseline(L, hidden, gpu_out, budget_s=12.0):
    """Times the CPU checker (single thread, as the reference's layer runs) on
    the same layer and tokens; repeats the forward until about budget_s of CPU
    work.  Host weights are replayed only for the experts the batch selects."""
    from oracle.binding import Oracle
    orc = Oracle()
    T = hidden.shape[0]
    pairs = orc.router(hidden, L.gate_w, L.gate_b, L.k)
    used = sorted(set(pairs[..., 0].astype(int).ravel().tolist()))
    per_gu, per_d = L.F * (L.H // 32) * 17, L.H * (L.F // 32) * 17
    wu = np.zeros(L.E * per_gu, np.uint8)
    wg = np.zeros(L.E * per_gu, np.uint8)
    wd = np.zeros(L.E * per_d, np.uint8)
    for e in used:
        wu[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 0)
        wg[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 1)
        wd[e * per_d:(e + 1) * per_d] = L.blocks(e, 2)
    args = (hidden, L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, wu, wg, wd, L.b_up, L.b_gate, L.b_down)
    # bounded sample: at most Tm tokens of the batch, repeated
    t0 = time.perf_counter()
    Tm = min(T, 4)
    ref, _ = orc.moe_layer(*args, max_tokens=Tm)
    first = time.perf_counter() - t0
    per_tok = first / Tm
    Tm = int(max(1, min(T, budget_s / max(per_tok, 1e-6))))
    reps = int(max(1, min(50, budget_s / (per_tok * Tm))))
    t0 = time.perf_counter()
    for _ in range(reps):
        ref, _ = orc.moe_layer(*args, max_tokens=Tm)
    dt = time.perf_counter() - t0
    err = float(np.max(np.abs(gpu_out[:Tm] - ref[:Tm])) / max(1e-6, np.max(np.abs(ref[:Tm]))))
    # not reference behaviour (its layer runs on one thread): the same work farmed over the
    # host's cores, one token slice per thread (the checker releases the GIL inside the call)
    ncores = max(1, min(16, os.cpu_count() or 1))
    all_cores = None
    if T >= ncores and ncores > 1:
        import threading
        per = max(1, min(T // ncores, max(1, int(budget_s / 2 / max(per_tok, 1e-6)))))
        slices = [np.ascontiguousarray(hidden[i * per:(i + 1) * per]) for i in range(ncores)]

        rounds = int(max(1, min(50, budget_s / 4 / max(per_tok * per, 1e-6))))

        def work(h):
            for _ in range(rounds):
                orc.moe_layer(h, *args[1:], max_tokens=h.shape[0])
        threads = [threading.Thread(target=work, args=(h,)) for h in slices]
        t0 = time.perf_counter()
        for th in threads:
            th.start()
        for th in threads:
            th.join()
        dt_all = time.perf_counter() - t0
        all_cores = dict(value=per * ncores * rounds / dt_all, unit="tokens/s", cores=ncores,
                         sample=f"{ncores} threads x {per} tokens x {rounds} rounds, {dt_all:.1f} s; "
                                f"not reference behaviour")
    return dict(value=Tm * reps / dt, unit="tokens/s", cores=1, kind="port", all_cores=all_cores,
                sample=f"first {Tm} of {T} tokens x {reps} repeats, {dt:.1f} s on one host core "
                       f"(CPU cost is linear in tokens x top_k)",
                gpu_vs_cpu_max_rel_err=err)


def cpu_baseline_f16(L, hidden, gpu_out, budget_s=12.0):
    """The CPU checker's fp16 expert path on the first tokens of the batch (the ones whose
    experts' generated weights were read back), one thread."""
    from oracle.binding import Oracle
    orc = Oracle()
    ns = L.f16_sample
    E, H, F = L.E, L.H, L.F
    w_up = np.zeros((E, F, H), np.float16)
    w_gate = np.zeros((E, F, H), np.float16)
    w_down = np.zeros((E, H, F), np.float16)
    for e, (u, g, d) in L.f16_weights.items():
        w_up[e], w_gate[e], w_down[e] = u, g, d
    args = (hidden[:ns], E, L.k, H, F, L.gate_w, L.gate_b, w_up, w_gate, w_down, L.b_up, L.b_gate, L.b_down)
    t0 = time.perf_counter()
    ref, _ = orc.moe_layer(*args)
    first = time.perf_counter() - t0
    reps = int(max(1, min(50, budget_s / max(first, 1e-6))))
    t0 = time.perf_counter()
    for _ in range(reps):
        ref, _ = orc.moe_layer(*args)
    dt = time.perf_counter() - t0
    err = float(np.max(np.abs(gpu_out[:ns] - ref)) / max(1e-6, np.max(np.abs(ref))))
    return dict(value=ns * reps / dt, unit="tokens/s", cores=1, kind="port", all_cores=None,
                sample=f"first {ns} of {hidden.shape[0]} tokens x {reps} repeats, {dt:.1f} s on one host core "
                       f"(CPU cost is linear in tokens x top_k)",
                gpu_vs_cpu_max_rel_err=err)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2_20b_decode", choices=sorted(SHAPES))
    ap.add_argument("--tokens", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="only the headline batch size")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run the 256 MiB copy kernel 10 times (known traffic, for profiler byte counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(no collectives, sharding or rank code are part of it).", file=sys.stderr)
        sys.exit(2)

    from coalsack_amd import load, synth
    lib = load(0)
    dev_name, cus, mem = lib.device_info()
    shape = SHAPES[a.workload]
    T = a.tokens or shape["default_T"]

    if a.workload == "gguf_ingest":
        res = bench_gguf_ingest(lib, synth, shape)
        line = dict(metric="GGUF MoE block ingest GB/s", value=res["file_bytes"] / res["seconds"] / 1e9,
                    unit="GB/s", n_gpus=1, steps=len(res["all_seconds"]), warmup=0,
                    ms_per_step=res["seconds"] * 1e3, higher_is_better=True, scaling="weak",
                    vs_baseline=None, dtype="u8", data="synthetic",
                    config=dict(workload="gguf_ingest: one 20b-shaped block (32 experts, MXFP4 + biases + router + norm) "
                                         "file -> resident layer", file_bytes=res["file_bytes"], device=dev_name),
                    roofline=None, cpu_baseline=None, roundtrip_ok=res["roundtrip_ok"], finite=res["finite"])
        print(json.dumps(line))
        return

    if a.workload == "c5_stack":
        res = bench_stack(lib, synth, shape, T, a.steps, a.warmup, shape["layers"])
        line = dict(metric="MoE stack tokens/s", value=res["tokens_per_s"], unit="tokens/s", n_gpus=1,
                    steps=a.steps, warmup=a.warmup, ms_per_step=res["ms_per_step"],
                    higher_is_better=True, scaling="weak", vs_baseline=None, dtype="mxfp4 x bf16(2-term) -> f32",
                    data="synthetic",
                    config=dict(workload=f"c5_stack: 36 x 120b-shaped MoE layer (RMSNorm + residual), T={T}",
                                tokens=T, device=dev_name,
                                distinct_experts_per_layer=res["distinct_experts_per_layer"]),
                    roofline=dict(bound="hbm", kernel="whole stack (all kernels of 36 layers)",
                                  achieved=res["stack_bytes"] / (res["ms_per_step"] * 1e-3) / 1e9,
                                  peak=HBM_PEAK_GBS, unit="GB/s", traffic=None,
                                  frac=res["stack_bytes"] / (res["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                  algorithmic_bytes=res["stack_bytes"]),
                    cpu_baseline=None, finite=res["finite"])
        print(json.dumps(line))
        return

    if a.calibrate:
        nbytes = 256 << 20
        src, dst = lib.dev_alloc(nbytes), lib.dev_alloc(nbytes)
        for _ in range(10):
            lib.copy_d2d(dst, src, nbytes)
        lib.synchronize()
        lib.dev_free(src)
        lib.dev_free(dst)
    res, (L, hidden, out) = bench_layer(lib, synth, shape, T, a.steps, a.warmup)
    prefill = T >= 512
    f16 = bool(shape.get("f16"))
    if f16 and prefill:
        st = res["stage_ms"]
        fl = T * shape["k"] * 4 * shape["H"] * shape["F"]
        roof = dict(bound="mfma", kernel="expert_f16_gemm_kernel<0> (gate/up + SwiGLU)", achieved=fl / (st["gateup"] * 1e-3) / 1e12,
                    peak=MFMA_F16_PEAK_TFLOPS, unit="TFLOP/s", traffic=None)
    elif f16:
        roof = dict(bound="hbm", kernel="expert_f16_kernel<0> (gate/up + SwiGLU)",
                    achieved=res["gateup_gbs"], peak=HBM_PEAK_GBS, unit="GB/s", traffic=None)
    elif prefill:
        st = res["stage_ms"]
        fl = T * shape["k"] * 4 * shape["H"] * shape["F"]  # gate + up flops
        roof = dict(bound="mfma", kernel="expert_gemm_mx_kernel<0> (gate/up + SwiGLU)", achieved=fl / (st["gateup"] * 1e-3) / 1e12,
                    peak=MFMA_FP4_PEAK_TFLOPS, unit="TFLOP/s", traffic=None)
    else:
        roof = dict(bound="hbm", kernel="expert_stream_kernel<2,*> (gate/up + SwiGLU)",
                    achieved=res["gateup_gbs"], peak=HBM_PEAK_GBS, unit="GB/s", traffic=None)
    # measured HBM traffic of that kernel, where a counter run has been recorded for this workload
    try:
        rec = json.load(open(os.path.join(ROOT, "profiles", "traffic.json"))).get(f"{a.workload}:T={T}")
    except (OSError, ValueError):
        rec = None
    if rec:
        roof["traffic"] = rec["bytes"]
        roof["traffic_source"] = rec["source"]
    roof["frac"] = roof["achieved"] / roof["peak"]
    if roof["bound"] == "hbm":
        roof["measured_copy_gbs"] = round(measured_copy_gbs(lib), 1)
        roof["frac_of_measured_copy"] = roof["achieved"] / roof["measured_copy_gbs"]
    roof["kernel_ms"] = res["stage_ms"]["gateup"]
    roof["algorithmic_bytes"] = res["gateup_bytes"]

    sweep = []
    if not a.no_sweep:
        for Ts in shape["sweep"]:
            if Ts == T:
                r = res
            else:
                r, _ = bench_layer(lib, synth, shape, Ts, max(20, a.steps // 2), a.warmup)
            sweep.append(dict(T=Ts, tokens_per_s=round(r["tokens_per_s"], 1), ms_per_step=round(r["ms_per_step"], 5),
                              distinct_experts=r["distinct_experts"], close_call_tokens=r["close_call_tokens"],
                              layer_hbm_frac=round(r["layer_hbm_frac"], 4),
                              gateup_hbm_frac=round(r["gateup_gbs"] / HBM_PEAK_GBS, 4),
                              stage_ms={kk: round(v, 5) for kk, v in r["stage_ms"].items()}))

    cpu = None if a.no_cpu else (cpu_baseline_f16(L, hidden, out) if f16 else cpu_baseline(L, hidden, out))
    line = dict(
        metric="MoE layer tokens/s", value=res["tokens_per_s"], unit="tokens/s", n_gpus=1, steps=res["steps"],
        warmup=a.warmup, ms_per_step=res["ms_per_step"], higher_is_better=True, scaling="weak",
        vs_baseline=None,
        dtype=("f16 x f16(2-term) -> f32" if f16 else
               "mxfp4 x fp6(3-term, block-scaled) -> f32" if prefill else "mxfp4 x bf16(2-term) -> f32"),
        data="synthetic",
        config=dict(workload=f"{a.workload}: E={shape['E']} top-{shape['k']} H={shape['H']} F={shape['F']} "
                             f"{'fp16' if f16 else 'MXFP4'}, T={T}" + (", 8 hot experts" if shape["hot"] else ""),
                    tokens=T, distinct_experts=res["distinct_experts"], token_batches_in_rotation=res["batches"],
                    close_call_tokens=res["close_call_tokens"], device=dev_name, compute_units=cus),
        roofline=roof, cpu_baseline=cpu,
        layer=dict(hbm_frac=res["layer_hbm_frac"], fp4_mfma_frac=res["layer_fp4_frac"],
                   algorithmic_bytes=res["layer_bytes"], algorithmic_flops=res["layer_flops"],
                   stage_ms=res["stage_ms"], finite=res["finite"]),
        sweep=sweep)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
