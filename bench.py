#!/usr/bin/env python3
"""Benchmark of the MoE layer (router -> dispatch -> MXFP4 expert MLP -> combine)
on one MI355X through the C ABI.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tokens T]

Prints ONE JSON line.  A step is one forward of the layer over one batch of T
synthetic tokens with weights, input and output resident in HBM.  `value` is
tokens/s of the whole layer; `roofline` describes the dominant kernel (gate/up
projections), timed live by a start and a stop event attached to its dispatch on
the library's stream (the kernel's own begin-to-end time, as a kernel trace
reports it); `cpu_baseline` is the CPU checker (a restatement of the
reference's single-threaded path) timed on this host on a bounded sample.

The default line is the 120b-shaped layer (128 experts, 8 hot) at 16 tokens and
carries, under `legs`, the same layer at 1 and at 4096 tokens and the 36-layer
stack at 1, 8 and 64 tokens, each with its own `roofline` and `cpu_baseline`.
Decode batches rotate over 8 layer instances x 8 token batches, so that no weight
byte is touched again before more than the 256 MB last-level cache has streamed by.

Workloads (BASELINE.json configs):
  c4_120b         128 experts, 8 hot experts (+2.0 router bias), T in {1,16,4096} (default, T=16)
  c2_20b_decode   32 experts, top-4, H = F = 2880, T in {1,2,4,8,16,32,64}
  c3_20b_prefill  same layer, T = 2048
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


def down_bytes(H, F, T, k, U, f16=False):
    """Algorithmic bytes of the down kernel: the matrix and bias of every distinct expert
    once, the activations in, one fp32 row per assignment out."""
    return U * (matrix_bytes(H, F, f16) + H * 4) + T * k * (F + H) * 4


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


def event_pair_overhead_ms(lib, reps=101):
    """What two consecutive event records with nothing between them read: the part of a
    `stage_ms` figure that is not the kernel."""
    vals = []
    for _ in range(reps):
        e0, e1 = lib.event(), lib.event()
        lib.record(e0)
        lib.record(e1)
        vals.append(lib.elapsed_ms(e0, e1))
        lib.dll.csk_event_destroy(e0)
        lib.dll.csk_event_destroy(e1)
    return float(np.median(vals))


def close_calls(L, hidden, k):
    """Tokens whose k+1 largest router logits contain two closer than the library's
    close-call threshold (8 * 2^-24 * sqrt(H), relative to max(1, |logit|)): those are
    recomputed in the reference's summation order, which costs tens of microseconds."""
    lg = hidden.astype(np.float64) @ L.gate_w.astype(np.float64).T + L.gate_b
    srt = -np.sort(-lg, axis=1)[:, :k + 1]
    gaps = (srt[:, :-1] - srt[:, 1:]) / np.maximum(1.0, np.abs(srt[:, :-1]))
    return int(np.count_nonzero(gaps.min(axis=1) <= 8 * 5.96e-8 * np.sqrt(hidden.shape[1])))


def bench_layer(lib, synth, shape, T, steps, warmup, seed=1234, layers=None):
    """Times exactly `steps` forwards.  Decode sizes rotate over nl layer instances x nb token
    batches (layer index fastest): the experts selected, and with them the bytes streamed,
    change from step to step, and a (layer, expert) pair comes back only after the other
    layers' traffic -- far more than the last-level cache holds -- has passed.
    `layers`: resident (LayerInputs, Layer) pairs to use instead of building new ones."""
    decode = T < 512
    nl, nb = (8, 8) if decode else (1, 1)
    own = layers is None
    if own:
        layers = [make_layer(lib, synth, shape, seed, layer_index=i) for i in range(nl)]
    layers = layers[:nl]
    nl = len(layers)
    L = layers[0][0]
    f16 = bool(shape.get("f16"))
    hiddens = [synth.hidden_states(T, L.H, seed=T + 1000 * i) for i in range(nb)]
    d_ins = [lib.to_device(h) for h in hiddens]
    d_out = lib.dev_alloc(hiddens[0].nbytes)
    ncombo = nl * nb
    turn = [0]

    def combo(i):
        return i % nl, (i // nl) % nb

    def fn():
        li, bi = combo(turn[0])
        layers[li][1].forward_device(d_ins[bi], T, d_out)
        turn[0] += 1
    ms = time_forward(lib, fn, steps, warmup)
    timed_combos = [combo(i) for i in range(warmup, warmup + steps)]

    # distinct experts of every combination (untimed)
    U, tmax = {}, 0
    for c in sorted(set(timed_combos) | {combo(i) for i in range(ncombo)}):
        layers[c[0]][1].forward_device(d_ins[c[1]], T, d_out)
        if T <= 32768:
            counts, _ = layers[c[0]][1].last_dispatch(T)
            U[c] = int(np.count_nonzero(counts))
            tmax = max(tmax, int(counts.max()))
        else:  # taken in several passes: no single dispatch to read back; every expert is in use
            U[c] = shape["E"]

    # per-stage and per-kernel times, every combination the same number of times
    rounds = max(1, min(6, 200 // ncombo))
    lib.stage_timing(True)
    stage_acc, kern_acc, have_kern, gu_bytes, dn_bytes = {}, [0.0, 0.0], not f16, 0, 0
    turn[0] = 0
    for _ in range(rounds * ncombo):
        c = combo(turn[0])
        fn()
        for kk, v in lib.stage_times().items():
            stage_acc[kk] = stage_acc.get(kk, 0.0) + v
        if have_kern:
            g, d = lib.kernel_times()
            kern_acc[0] += g
            kern_acc[1] += d
        gu_bytes += gateup_bytes(L.H, L.F, T, L.k, U[c], f16)
        dn_bytes += down_bytes(L.H, L.F, T, L.k, U[c], f16)
    lib.stage_timing(False)
    n_prof = rounds * ncombo
    stages = {kk: v / n_prof for kk, v in stage_acc.items()}
    kernels = dict(gateup=kern_acc[0] / n_prof, down=kern_acc[1] / n_prof) if have_kern else None

    # combination (0, 0) last: its output is the one checked against the CPU path
    layers[0][1].forward_device(d_ins[0], T, d_out)
    hidden = hiddens[0]
    out = lib.to_host(d_out, (T, L.H))
    L.f16_weights = None
    if f16:
        # the CPU leg needs the generated halves of the experts its token sample selects
        from coalsack_amd import capi
        ns = min(T, 2)
        _, pairs = layers[0][1].forward(hidden[:ns], want_pairs=True)
        L.f16_weights = {int(e): [layers[0][1].export_f16(int(e), w) for w in (capi.W_UP, capi.W_GATE, capi.W_DOWN)]
                         for e in sorted(set(pairs[..., 0].astype(int).ravel().tolist()))}
        L.f16_sample = ns
    for d in d_ins:
        lib.dev_free(d)
    lib.dev_free(d_out)
    if own:
        for _, layer in layers:
            layer.close()
    U_timed = float(np.mean([U[c] for c in timed_combos]))
    res = dict(T=T, ms_per_step=ms, tokens_per_s=T / (ms * 1e-3), distinct_experts=U_timed,
               stage_ms=stages, kernel_ms=kernels, finite=bool(np.all(np.isfinite(out))),
               max_tokens_per_expert=tmax, batches=nb, layer_instances=nl, steps=steps,
               close_call_tokens=sum(close_calls(layers[0][0], h, L.k) for h in hiddens))
    res["layer_bytes"] = float(np.mean([layer_bytes(L.E, L.k, L.H, L.F, T, U[c], f16) for c in timed_combos]))
    res["layer_hbm_frac"] = res["layer_bytes"] / (ms * 1e-3) / (HBM_PEAK_GBS * 1e9)
    res["layer_flops"] = layer_flops(L.E, L.k, L.H, L.F, T)
    res["layer_fp4_frac"] = res["layer_flops"] / (ms * 1e-3) / (MFMA_FP4_PEAK_TFLOPS * 1e12)
    res["gateup_bytes"] = gu_bytes / n_prof
    res["down_bytes"] = dn_bytes / n_prof
    res["gateup_ms"] = kernels["gateup"] if kernels else stages["gateup"]
    res["gateup_gbs"] = res["gateup_bytes"] / (res["gateup_ms"] * 1e-3) / 1e9
    res["rotation"] = [(layers[i][0], hiddens[i % nb]) for i in range(nl)]
    return res, (L, hidden, out)


def layer_roofline(res, shape, T, workload):
    """`roofline` object of a layer measurement: its gate/up kernel."""
    prefill = T >= 512
    f16 = bool(shape.get("f16"))
    fl = T * shape["k"] * 4 * shape["H"] * shape["F"]  # gate + up flops
    clock = ("start/stop events on the kernel's dispatch (begin-to-end, as a kernel trace reports it)"
             if res["kernel_ms"] else "events recorded around the launch")
    if prefill:
        roof = dict(bound="mfma",
                    kernel=("expert_f16_gemm_kernel<0>" if f16 else "expert_gemm_mx_kernel<0>") + " (gate/up + SwiGLU)",
                    achieved=fl / (res["gateup_ms"] * 1e-3) / 1e12,
                    peak=MFMA_F16_PEAK_TFLOPS if f16 else MFMA_FP4_PEAK_TFLOPS, unit="TFLOP/s", traffic=None,
                    algorithmic_flops=fl)
    else:
        roof = dict(bound="hbm",
                    kernel=("expert_f16_kernel<0>" if f16 else "expert_stream_kernel<0,*>") +
                    (" (top-k routing of the one token + gate/up + SwiGLU: no routing launch in front)"
                     if (T == 1 and not f16) else " (gate/up + SwiGLU)"),
                    achieved=res["gateup_gbs"], peak=HBM_PEAK_GBS, unit="GB/s", traffic=None,
                    algorithmic_bytes=res["gateup_bytes"])
    # HBM traffic of that kernel from a recorded counter run of this workload, where there is one
    try:
        rec = json.load(open(os.path.join(ROOT, "profiles", "traffic.json"))).get(f"{workload}:T={T}")
    except (OSError, ValueError):
        rec = None
    if rec:
        roof["traffic"] = rec["bytes"]
        roof["traffic_source"] = rec["source"] + " (a recorded counter run, not measured in this run)"
    roof["frac"] = roof["achieved"] / roof["peak"]
    if prefill and not f16:
        # every product is issued three times (three FP6 activation terms meet the 1e-3 bar, two do not):
        # the algorithmic rate cannot exceed a third of the FP6 x FP4 peak
        roof["three_term_cap"] = roof["peak"] / 3
        roof["frac_of_three_term_cap"] = roof["achieved"] / roof["three_term_cap"]
    roof["kernel_ms"] = res["gateup_ms"]
    roof["kernel_clock"] = clock
    if res["kernel_ms"]:
        roof["down_kernel_ms"] = res["kernel_ms"]["down"]
        if prefill:
            roof["down_achieved"] = fl / 2 / (res["kernel_ms"]["down"] * 1e-3) / 1e12
        else:
            roof["down_algorithmic_bytes"] = res["down_bytes"]
            roof["down_achieved"] = res["down_bytes"] / (res["kernel_ms"]["down"] * 1e-3) / 1e9
        roof["down_frac"] = roof["down_achieved"] / roof["peak"]
    return roof


def bench_stack(lib, synth, shape, T, steps, warmup, layers):
    """36 resident layers, h <- h + MoE(RMSNorm(h)) each; `layers` = (LayerInputs, Layer) pairs."""
    from coalsack_amd.capi import stack_forward, FWD_RMSNORM, FWD_RESIDUAL
    handles = [layer for _, layer in layers]
    hidden = synth.hidden_states(T, shape["H"], seed=T)
    d_h = lib.to_device(hidden)
    d_h0 = lib.to_device(hidden)

    def fn():
        # the stack updates the hidden states in place; start every step from the same N(0,1) input
        lib.copy_d2d(d_h, d_h0, hidden.nbytes)
        stack_forward(lib, handles, d_h, T)
    ms = time_forward(lib, fn, steps, warmup)
    out = lib.to_host(d_h, hidden.shape)
    # untimed pass, layer by layer: distinct experts each layer streams, and the kernels' own times
    lib.copy_d2d(d_h, d_h0, hidden.nbytes)
    lib.stage_timing(True)
    total_bytes, distinct, gu_bytes, gu_ms, dn_ms, side_ms = 0, [], 0, 0.0, 0.0, 0.0
    first_out = None
    for layer in handles:
        layer.forward_device(d_h, T, d_h, FWD_RMSNORM | FWD_RESIDUAL)
        if first_out is None:
            first_out = lib.to_host(d_h, hidden.shape)
        st = lib.stage_times()
        g, d = lib.kernel_times()
        counts, _ = layer.last_dispatch(T)
        U = int(np.count_nonzero(counts))
        distinct.append(U)
        total_bytes += layer_bytes(shape["E"], shape["k"], shape["H"], shape["F"], T, U) + shape["H"] * 4
        gu_bytes += gateup_bytes(shape["H"], shape["F"], T, shape["k"], U)
        gu_ms += g
        dn_ms += d
        side_ms += st["prep"] + st["router"] + st["dispatch"] + st["combine"]
    lib.stage_timing(False)
    lib.dev_free(d_h)
    lib.dev_free(d_h0)
    return dict(T=T, layers=len(handles), ms_per_step=ms, tokens_per_s=T / (ms * 1e-3),
                finite=bool(np.all(np.isfinite(out))), stack_bytes=total_bytes,
                distinct_experts_per_layer=distinct, gateup_bytes=gu_bytes, gateup_ms=gu_ms, down_ms=dn_ms,
                side_stage_ms=side_ms, hidden=hidden, first_layer_out=first_out)


def stack_roofline(res):
    frac = res["stack_bytes"] / (res["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS
    return dict(bound="hbm", kernel="whole stack (all kernels of 36 layers)",
                achieved=frac * HBM_PEAK_GBS, peak=HBM_PEAK_GBS, unit="GB/s", traffic=None, frac=frac,
                algorithmic_bytes=res["stack_bytes"],
                gateup_kernels=dict(ms=res["gateup_ms"], algorithmic_bytes=res["gateup_bytes"],
                                    frac=res["gateup_bytes"] / (res["gateup_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                    clock="start/stop events on each dispatch, summed over the 36 layers"),
                down_kernels_ms=res["down_ms"], side_stages_ms_with_event_overhead=res["side_stage_ms"])


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


def host_cpu():
    """Model string and last-level cache of the host the CPU baseline runs on."""
    model, llc = "unknown", 0
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name"):
                model = ln.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        base = "/sys/devices/system/cpu/cpu0/cache"
        for idx in sorted(os.listdir(base)):
            sz = open(os.path.join(base, idx, "size")).read().strip()
            val = int(sz[:-1]) * (1 << 10 if sz[-1] == "K" else 1 << 20) if sz[-1] in "KM" else int(sz)
            llc = max(llc, val)
    except (OSError, ValueError):
        pass
    return model, llc


def cpu_baseline(insts, gpu_out, budget_s=12.0, stack_layers=0):
    """Times the CPU checker (single thread, as the reference's layer runs) on the same
    layers and tokens.  `insts`: (LayerInputs, hidden) pairs -- the layer instances and token
    batches the GPU measurement rotates over; gpu_out is the GPU's output for insts[0].

    One definition for every leg: `value` is the COLD rate -- the sample walks distinct
    tokens (and, where one batch selects too few experts, distinct layer instances) so that
    the expert slices a token reads (4 x 13 MB) have not been touched since more than the
    host's last-level cache has streamed by, which is how the reference meets them in a
    model of 36 layers.  `warm` is the same work with the sample small enough to be re-read
    from cache (one token repeated), reported beside it.  Only the tokens that are timed
    are handed to the checker (its router runs over every token it is given).
    stack_layers > 0: each instance is a layer of a stack of that many (RMSNorm in front,
    residual add behind); the stack's rate is the layer's divided by the number of layers."""
    from oracle.binding import Oracle
    orc = Oracle()
    stack = stack_layers > 0
    model, llc = host_cpu()
    llc = llc or (256 << 20)
    L0, hidden0 = insts[0]
    T = hidden0.shape[0]
    per_gu, per_d = L0.F * (L0.H // 32) * 17, L0.H * (L0.F // 32) * 17
    slice_bytes = 2 * per_gu + per_d
    t_gen0 = time.perf_counter()
    # token sample: at most 32 tokens per instance (replaying an expert's generated bytes on the
    # host costs ~0.1 s), instances added until the experts they select exceed 4 x the LLC
    Ts = min(T, 32)
    work, ws_bytes = [], 0
    for L, hidden in insts:
        h = np.ascontiguousarray(hidden[:Ts])
        pairs = orc.router(orc.rmsnorm(h, L.norm_w, 1e-5) if stack else h, L.gate_w, L.gate_b, L.k)
        used = sorted(set(pairs[..., 0].astype(int).ravel().tolist()))
        wu = np.zeros(L.E * per_gu, np.uint8)  # (untouched pages of absent experts cost no memory)
        wg = np.zeros(L.E * per_gu, np.uint8)
        wd = np.zeros(L.E * per_d, np.uint8)
        for e in used:
            wu[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 0)
            wg[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 1)
            wd[e * per_d:(e + 1) * per_d] = L.blocks(e, 2)
        kw = dict(norm_w=L.norm_w, norm_eps=1e-5, residual=True) if stack else {}
        work.append((h, (L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, wu, wg, wd, L.b_up, L.b_gate, L.b_down), kw))
        ws_bytes += len(used) * slice_bytes
        if ws_bytes > 4 * llc:
            break
    gen_s = time.perf_counter() - t_gen0

    def run(i, lo, hi):
        h, args, kw = work[i]
        return orc.moe_layer(np.ascontiguousarray(h[lo:hi]), *args, **kw)[0]

    # parity of the GPU's output on the sample of instance 0 (also the first touch of its pages)
    ref = run(0, 0, Ts)
    err = float(np.max(np.abs(gpu_out[:Ts] - ref)) / max(1e-6, np.max(np.abs(ref))))
    # cold: one token at a time, instances interleaved, until the budget is spent
    order = [(i, t) for t in range(Ts) for i in range(len(work))]
    n, t0 = 0, time.perf_counter()
    while True:
        for i, t in order:
            run(i, t, t + 1)
            n += 1
            if time.perf_counter() - t0 > budget_s * 0.7:
                break
        else:
            continue
        break
    dt_cold = time.perf_counter() - t0
    cold = n / dt_cold
    # warm: token 0 of instance 0 over and over (4 expert slices, 53 MB)
    m, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s * 0.15 or m < 3:
        run(0, 0, 1)
        m += 1
    warm = m / (time.perf_counter() - t0)
    # not reference behaviour (its layer runs on one thread): the same work farmed over the
    # host's cores, one token slice per thread (the checker releases the GIL inside the call)
    ncores = max(1, min(16, os.cpu_count() or 1))
    all_cores = None
    if Ts >= ncores and ncores > 1:
        import threading
        per = Ts // ncores
        rounds = int(max(1, min(50, budget_s * 0.15 * cold * ncores / (per * ncores))))

        def farm(j):
            for _ in range(rounds):
                run(0, j * per, (j + 1) * per)
        threads = [threading.Thread(target=farm, args=(j,)) for j in range(ncores)]
        t0 = time.perf_counter()
        for th in threads:
            th.start()
        for th in threads:
            th.join()
        dt_all = time.perf_counter() - t0
        all_cores = dict(value=per * ncores * rounds / dt_all / max(1, stack_layers), unit="tokens/s", cores=ncores,
                         sample=f"{ncores} threads x {per} tokens x {rounds} rounds, {dt_all:.1f} s; "
                                f"not reference behaviour")
    div = max(1, stack_layers)
    return dict(value=cold / div, unit="tokens/s", cores=1, kind="port", host_cpu=model,
                host_llc_bytes=llc, warm=dict(value=warm / div, unit="tokens/s",
                                              sample=f"token 0 of instance 0 repeated {m} times: its 4 expert slices "
                                                     f"({4 * slice_bytes / 1e6:.0f} MB) are re-read from cache where the "
                                                     f"last-level cache ({llc / 2**20:.0f} MiB) holds them"),
                all_cores=all_cores,
                sample=f"cold: {n} single-token forwards in {dt_cold:.1f} s on one host core, walking the first {Ts} of "
                       f"{T} tokens of {len(work)} layer instance(s) in turn: {ws_bytes / 1e6:.0f} MB of expert slices "
                       f"pass between two uses of the same one (CPU cost is linear in tokens x top_k); "
                       f"{gen_s:.1f} s of host weight replay not counted"
                       + (f"; layers of the stack (RMSNorm + MoE + residual), rate divided by {stack_layers} "
                          f"layers of identical shape" if stack else ""),
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


def layer_leg(lib, synth, shape, workload, T, steps, warmup, layers, cpu, budget_s):
    """One measured (workload, T) of a single layer as a JSON-able object."""
    res, (L, hidden, out) = bench_layer(lib, synth, shape, T, steps, warmup, layers=layers)
    leg = dict(workload=f"{workload} T={T}", tokens=T, value=res["tokens_per_s"], unit="tokens/s",
               ms_per_step=res["ms_per_step"], steps=res["steps"], distinct_experts=res["distinct_experts"],
               close_call_tokens=res["close_call_tokens"],
               roofline=layer_roofline(res, shape, T, workload),
               layer=dict(hbm_frac=res["layer_hbm_frac"], fp4_mfma_frac=res["layer_fp4_frac"],
                          algorithmic_bytes=res["layer_bytes"], algorithmic_flops=res["layer_flops"],
                          stage_ms={kk: round(v, 5) for kk, v in res["stage_ms"].items()},
                          finite=res["finite"]),
               cpu_baseline=((cpu_baseline_f16(L, hidden, out, budget_s) if shape.get("f16") else
                              cpu_baseline(res["rotation"], out, budget_s)) if cpu else None))
    return leg, res, (L, hidden, out)


def stack_leg(lib, synth, shape, T, steps, warmup, layers, cpu, budget_s):
    res = bench_stack(lib, synth, shape, T, steps, warmup, layers)
    return dict(workload=f"c5_stack: {len(layers)} x 120b-shaped MoE layer (RMSNorm + residual) T={T}", tokens=T,
                value=res["tokens_per_s"], unit="tokens/s", ms_per_step=res["ms_per_step"], steps=steps,
                distinct_experts_per_layer=res["distinct_experts_per_layer"], finite=res["finite"],
                roofline=stack_roofline(res),
                cpu_baseline=(cpu_baseline([(Li, res["hidden"]) for Li, _ in layers[:8]], res["first_layer_out"],
                                           budget_s, stack_layers=len(layers)) if cpu else None))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c4_120b", choices=sorted(SHAPES))
    ap.add_argument("--tokens", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-sweep", action="store_true", help="only the headline batch size (no sweep)")
    ap.add_argument("--no-legs", action="store_true",
                    help="c4_120b: only the headline measurement, none of the other north-star legs")
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

    if a.calibrate:
        nbytes = 256 << 20
        src, dst = lib.dev_alloc(nbytes), lib.dev_alloc(nbytes)
        for _ in range(10):
            lib.copy_d2d(dst, src, nbytes)
        lib.synchronize()
        lib.dev_free(src)
        lib.dev_free(dst)

    is120 = a.workload in ("c4_120b", "c5_stack")
    legs_wanted = a.workload == "c4_120b" and not a.no_legs and not a.tokens
    # resident layers of the 120b shape: 36 for the stack legs, 8 for a decode rotation, 1 for prefill
    n_res = 36 if (a.workload == "c5_stack" or legs_wanted) else (8 if T < 512 else 1)
    layers120 = None
    if is120:
        layers120 = [make_layer(lib, synth, SHAPES["c5_stack"], 1234, layer_index=i, norm=True) for i in range(n_res)]

    if a.workload == "c5_stack":
        leg = stack_leg(lib, synth, shape, T, a.steps, a.warmup, layers120, not a.no_cpu, 12.0)
        line = dict(metric="MoE stack tokens/s", value=leg["value"], unit="tokens/s", n_gpus=1,
                    steps=a.steps, warmup=a.warmup, ms_per_step=leg["ms_per_step"],
                    higher_is_better=True, scaling="weak", vs_baseline=None, dtype="mxfp4 x fp6(3-term, block-scaled) -> f32",
                    data="synthetic",
                    config=dict(workload=leg["workload"], tokens=T, device=dev_name,
                                distinct_experts_per_layer=leg["distinct_experts_per_layer"]),
                    roofline=leg["roofline"], cpu_baseline=leg["cpu_baseline"], finite=leg["finite"])
        print(json.dumps(line))
        return

    head, res, (L, hidden, out) = layer_leg(lib, synth, shape, a.workload, T, a.steps, a.warmup, layers120,
                                            not a.no_cpu, 12.0)
    prefill = T >= 512
    f16 = bool(shape.get("f16"))
    roof = head["roofline"]
    if roof["bound"] == "hbm":
        roof["measured_copy_gbs"] = round(measured_copy_gbs(lib), 1)
        roof["frac_of_measured_copy"] = roof["achieved"] / roof["measured_copy_gbs"]
    roof["event_pair_overhead_ms"] = round(event_pair_overhead_ms(lib), 5)

    sweep = []
    if not a.no_sweep and not legs_wanted:
        for Ts in shape["sweep"]:
            if Ts == T:
                r = res
            else:
                r, _ = bench_layer(lib, synth, shape, Ts, max(20, a.steps // 2), a.warmup, layers=layers120)
            sweep.append(dict(T=Ts, tokens_per_s=round(r["tokens_per_s"], 1), ms_per_step=round(r["ms_per_step"], 5),
                              distinct_experts=r["distinct_experts"], close_call_tokens=r["close_call_tokens"],
                              layer_hbm_frac=round(r["layer_hbm_frac"], 4),
                              gateup_hbm_frac=round(r["gateup_gbs"] / HBM_PEAK_GBS, 4),
                              stage_ms={kk: round(v, 5) for kk, v in r["stage_ms"].items()}))

    legs = []
    if legs_wanted:
        # the other configurations the target is stated on, in the same line
        cpu = not a.no_cpu
        legs.append(layer_leg(lib, synth, shape, "c4_120b", 1, a.steps, a.warmup, layers120, cpu, 8.0)[0])
        legs.append(layer_leg(lib, synth, shape, "c4_120b", 4096, max(10, a.steps // 10), max(3, a.warmup // 5),
                              layers120, cpu, 8.0)[0])
        for Ts in SHAPES["c5_stack"]["sweep"]:
            legs.append(stack_leg(lib, synth, SHAPES["c5_stack"], Ts, max(10, a.steps // 10), max(3, a.warmup // 5),
                                  layers120, cpu, 8.0))

    def leg_summary(leg):
        r, c = leg["roofline"], leg.get("cpu_baseline")
        out = dict(tokens_per_s=round(leg["value"], 1), ms_per_step=round(leg["ms_per_step"], 5), bound=r["bound"],
                   frac=round(r["frac"], 4), cpu_tokens_per_s=round(c["value"], 2) if c else None)
        if "kernel_ms" in r:
            out["kernel_ms"] = round(r["kernel_ms"], 5)
        if "down_frac" in r:
            out["down_frac"] = round(r["down_frac"], 4)
        if "frac_of_three_term_cap" in r:
            out["frac_of_three_term_cap"] = round(r["frac_of_three_term_cap"], 4)
        if "layer" in leg:
            out["layer_frac"] = round(leg["layer"]["fp4_mfma_frac" if r["bound"] == "mfma" else "hbm_frac"], 4)
        return out
    if legs:
        # the north-star legs in short, inside the object that describes the dominant kernel
        # (the long per-leg objects stay under `legs`)
        roof["legs"] = {"T1": leg_summary(legs[0]), "T4096": leg_summary(legs[1]),
                        "stack": {f"T{lg['tokens']}": leg_summary(lg) for lg in legs[2:]}}

    line = dict(
        metric="MoE layer tokens/s", value=head["value"], unit="tokens/s", n_gpus=1, steps=res["steps"],
        warmup=a.warmup, ms_per_step=head["ms_per_step"], higher_is_better=True, scaling="weak",
        vs_baseline=None,
        dtype=("f16 x f16(2-term) -> f32" if f16 else
               "mxfp4 x fp6(3-term, block-scaled) -> f32"),
        data="synthetic",
        config=dict(workload=f"{a.workload}: E={shape['E']} top-{shape['k']} H={shape['H']} F={shape['F']} "
                             f"{'fp16' if f16 else 'MXFP4'}, T={T}" + (", 8 hot experts" if shape["hot"] else ""),
                    tokens=T, distinct_experts=res["distinct_experts"],
                    rotation=f"{res['layer_instances']} layer instances x {res['batches']} token batches",
                    close_call_tokens=res["close_call_tokens"], device=dev_name, compute_units=cus),
        roofline=roof, cpu_baseline=head["cpu_baseline"], layer=head["layer"], sweep=sweep, legs=legs)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
