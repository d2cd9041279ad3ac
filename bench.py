#!/usr/bin/env python3
"""WKV6 forward+backward throughput on one MI355X, with roofline and CPU baseline.

One "step" = one forward + one backward of the WKV6 operator over one batch of synthetic input
at the RWKV6-1.6B layer shape (B=8, T=1024, C=2048, H=32, N=64, bf16 I/O, fp32 state), inputs
resident in HBM, outputs and workspace pre-allocated, called through the C ABI of
libwkv6_gfx950.so on torch's current stream, gu batch-sum included.

Prints ONE JSON line.  `--gpus N` with N > 1 is refused: this operator has no cross-GPU part
(every (batch, head) pair is independent), and this build measures a single GPU.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "star-rwkv6_amd"))
os.environ.setdefault("KERAS_BACKEND", "torch")

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOADS = {
    # name: (B, T, H, dtype)
    "c2": (8, 1024, 32, "bf16"),   # RWKV6-1.6B layer shape: the configuration the metric is quoted on
    "c3": (4, 4096, 64, "bf16"),   # RWKV6-7B layer shape
    "c1": (2, 128, 4, "f32"),
    "c2_f32": (8, 1024, 32, "f32"),   # the c2 shape with fp32 tensors (the full-precision chunk form; --algo scan: per-timestep kernels)
    "c2_f16": (8, 1024, 32, "f16"),   # ... with fp16 tensors: y, gy and the gradients are fp32 (--algo chunk: the bf16-operand pair)
    "long1": (1, 8192, 32, "bf16"),   # one long sequence per GPU (fine-tuning): 32 pairs, runs as time segments
    "short": (128, 256, 32, "bf16"),  # many short sequences: 4096 pairs, every workgroup takes 16 of them back to back
}

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (separate runs), scaled
# by the same counters' reading for a device-to-device copy of known size; see profiles/.
# Keyed by (workload, algo, "fwd"|"bwd").  None = not measured.
MEASURED_TRAFFIC_BYTES = {
    # profiles/c2_fwd_bwd_hbm_traffic_pmc.md: backward_saved_sum 201.8 MB read + 135.8 MB written,
    # forward_save 134.5 MB read + 67.1 MB written
    ("c2", "auto", "bwd"): 337.5e6, ("c2", "chunk", "bwd"): 337.5e6,
    ("c2", "auto", "fwd"): 201.6e6, ("c2", "chunk", "fwd"): 201.6e6,
    # profiles/c2_f32_fwd_bwd_kernel_trace.md: backward 470.3 MB read + 268.5 MB written, forward 268.8 + 201.3 MB
    ("c2_f32", "auto", "bwd"): 738.8e6, ("c2_f32", "auto", "fwd"): 470.1e6,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--preheat-ms", type=float, default=600.0,
                    help="untimed run of the same step before --warmup, so that the clocks are up whatever --warmup is")
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS) + ["c4", "c5", "mix"])
    ap.add_argument("--algo", default="auto", choices=["auto", "scan", "chunk"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-timings", action="store_true",
                    help="skip the unstaggered and the through-the-binding steps (profiles of the headline step alone)")
    ap.add_argument("--plain-pair", action="store_true", help="time forward()+backward() without saved states")
    ap.add_argument("--cpu-tokens", type=int, default=0, help="tokens in the CPU baseline sample (0 = default)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--stagger", type=int, default=256,
                    help="bytes by which each tensor's base is shifted against the one before (0: all 2 MiB-aligned)")
    return ap.parse_args()


def synthetic_inputs(B, T, H, N, seed, with_state=False):
    """The workload's seeded distributions, drawn on the CPU in float32: r, k, v ~ N(0,1);
    w = x ~ U(-6,1) passed raw (the operator applies exp(-exp(w))); u ~ N(0,0.5^2) (H,N); gy ~ N(0,1);
    with_state: h0 ~ N(0,0.1^2) (B,H,N,N)."""
    import torch

    g = torch.Generator().manual_seed(seed)
    C = H * N
    r, k, v = (torch.randn(B, T, C, generator=g) for _ in range(3))
    w = torch.rand(B, T, C, generator=g) * 7.0 - 6.0
    u = torch.randn(H, N, generator=g) * 0.5
    out = [r, k, v, w, u, torch.randn(B, T, C, generator=g)]
    if with_state:
        out.append(torch.randn(B, H, N, N, generator=g) * 0.1)
    return out


def preheat(step, ms):
    """Runs `step` untimed for about `ms` milliseconds (the GPU's clocks come up over the first
    few hundred milliseconds of load); returns the milliseconds spent."""
    import torch

    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(50):
            step()
        torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3


def cpu_baseline(B, T_full, H, N, seed, tokens):
    """The reference's python loop (restated in oracle/wkv6_ref.py) forward + autograd backward,
    fp32, all host cores, on a bounded sample of the same workload: same B, C and input
    distributions, fewer timesteps (cost is linear in T).  The sample doubles until it has taken
    about 10 s (or reaches the full T)."""
    import torch
    from oracle import wkv6_ref

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    Ts = max(8, min(T_full, (tokens or 512) // B))
    while True:
        r, k, v, w, u, gy = wkv6_ref.make_inputs(B, Ts, H, N, seed)
        t0 = time.perf_counter()
        leaves = [x.clone().requires_grad_(True) for x in (r, k, v, w, u)]
        y, _ = wkv6_ref.loop_torch(*leaves, N)
        y.backward(gy)
        dt = time.perf_counter() - t0
        del leaves, y
        if tokens or dt >= 8.0 or Ts >= T_full:
            break
        Ts = min(T_full, Ts * (2 if dt > 2.0 else 4))
    return {
        "value": B * Ts / dt / 1e6, "unit": "Mtokens/s", "cores": cores, "kind": "port",
        "sample": "python-loop WKV6 fwd+bwd via torch.autograd, fp32, B=%d T=%d of %d C=%d (%.1f s)" % (
            B, Ts, T_full, H * N, dt),
    }


def bench_stateful(a):
    """Config 5: B=64 sequences at C=2048, chunked prefill of T=512 from h0 then 256 single-token
    steps carrying the fp32 state, through the C ABI with pre-allocated buffers.  Prints its own JSON
    line (prefill Mtokens/s, decode steps/s and the state bandwidth of a decode step)."""
    import torch
    from rwkv_kernel import _native

    lib = _native.load()
    B, H, N, Tp, Td = 64, 32, 64, 512, 256
    C = H * N
    dev = torch.device("cuda:0")
    ins = synthetic_inputs(B, Tp + 1, H, N, a.seed, with_state=True)
    r, k, v, w, u = (x.to(torch.bfloat16).to(dev) for x in ins[:5])
    h0 = ins[6].to(dev)
    pre = [x[:, :Tp].contiguous() for x in (r, k, v, w)]
    one = [x[:, Tp:].contiguous() for x in (r, k, v, w)]
    yp = torch.empty(B, Tp, C, dtype=torch.bfloat16, device=dev)
    y1 = torch.empty(B, 1, C, dtype=torch.bfloat16, device=dev)
    sa, sb = torch.empty_like(h0), torch.empty_like(h0)
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()

    def call(x, T, y, si, so):
        _native.check(lib.wkv6_forward_with_state_ex(st, _native.BF16, _native.F32, _native.ALGO_AUTO, B, T, C, H, 1, None,
                                                     P(x[0]), P(x[1]), P(x[2]), P(x[3]), P(u), P(si), P(y), P(so), None, 0))

    def timed(fn, reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(max(1, a.warmup)):   # untimed: brings the clocks up as in a running service
            fn()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record(); torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    pre_ms = timed(lambda: call(pre, Tp, yp, h0, sa), 20)
    # the same prefill with the layer's group norm and gate fused into the kernel's output stage
    gate = torch.randn(B, Tp, C, device=dev).to(torch.bfloat16)
    gn_scale, gn_offset = torch.ones(H, N, device=dev), torch.zeros(H, N, device=dev)
    fused_ms = timed(lambda: _native.check(lib.wkv6_forward_gn_gate(
        st, _native.BF16, _native.F32, B, Tp, C, H, 1, None, P(pre[0]), P(pre[1]), P(pre[2]), P(pre[3]), P(u), P(h0),
        P(gate), P(gn_scale), P(gn_offset), 64e-5, P(yp), P(sa))), 20)

    # one long sequence alone on the chip (B=1, T=4096): as one pass, and as time segments side by
    # side (what the optional forward workspace enables)
    T1 = 4096
    g1 = torch.Generator().manual_seed(a.seed + 1)
    solo = [torch.randn(1, T1, C, generator=g1).to(torch.bfloat16).to(dev) for _ in range(3)]
    solo.append((torch.rand(1, T1, C, generator=g1) * 7 - 6).to(torch.bfloat16).to(dev))
    solo = [solo[0], solo[1], solo[2], solo[3]]
    y_solo = torch.empty(1, T1, C, dtype=torch.bfloat16, device=dev)
    s_solo, s_solo_out = h0[:1].contiguous(), torch.empty_like(h0[:1])
    n_ws = int(lib.wkv6_forward_workspace_bytes(_native.BF16, _native.ALGO_AUTO, 1, T1, C, H))
    ws = torch.empty(max(n_ws, 16), dtype=torch.uint8, device=dev)

    def solo_call(use_ws):
        _native.check(lib.wkv6_forward_with_state_ex(st, _native.BF16, _native.F32, _native.ALGO_AUTO, 1, T1, C, H, 1, None,
                                                     P(solo[0]), P(solo[1]), P(solo[2]), P(solo[3]), P(u), P(s_solo), P(y_solo),
                                                     P(s_solo_out), P(ws) if use_ws else None, n_ws if use_ws else 0))

    solo_one_ms = timed(lambda: solo_call(False), 20)
    solo_seg_ms = timed(lambda: solo_call(True), 20) if n_ws else None

    def two_steps():
        call(one, 1, y1, sa, sb); call(one, 1, y1, sb, sa)

    dec_ms = timed(two_steps, Td // 2) / 2
    state_bytes = 2 * B * H * N * N * 4
    print(json.dumps({
        "metric": "WKV6 stateful forward, B64 C2048 H32 bf16 activations, fp32 state", "n_gpus": 1,
        "config": {"workload": "c5: prefill T=512 then T=1 decode steps with carried state"},
        "prefill_Mtokens_per_s": B * Tp / (pre_ms * 1e-3) / 1e6, "prefill_ms": pre_ms,
        "prefill_with_group_norm_and_gate_ms": fused_ms,
        "single_sequence_prefill": {"B": 1, "T": T1, "one_pass_ms": solo_one_ms, "in_time_segments_ms": solo_seg_ms},
        "decode_steps_per_s": 1.0 / (dec_ms * 1e-3), "decode_us_per_step": dec_ms * 1e3,
        "decode_state_GBps": state_bytes / (dec_ms * 1e-3) / 1e9,
        "decode_frac_of_hbm_peak": state_bytes / (dec_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "dtype": "bf16", "data": "synthetic"}))


def bench_model_step(a):
    """Config 4: one full RWKV-6 training step (24 layers, d_model 2048, 32 heads of 64, FFN 7168,
    vocab 65536, random init, bf16 autocast, 8 x 1024 uniform random token ids, next-token cross
    entropy, forward + backward + AdamW) through the torch binding of the operator.  Prints its own
    JSON line: whole-step tokens/s and the share of the step spent inside the operator."""
    import torch
    import rwkv6_harness as hz
    from rwkv_kernel import RWKVKernelOperator

    dev = torch.device("cuda:0")
    torch.manual_seed(a.seed)
    B, T = 8, 1024
    model = hz.RWKV6(RWKVKernelOperator(64, T), **hz.CONFIG4).to(dev)
    opt = torch.optim.AdamW(model.parameters(), lr=1e-4, fused=True)
    ids = torch.randint(0, hz.CONFIG4["vocabulary_size"], (B, T + 1), device=dev)
    steps, warm = min(a.steps, 10), min(a.warmup, 3)
    losses = [float(hz.train_step(model, opt, ids, torch.bfloat16)) for _ in range(warm)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = hz.train_step(model, opt, ids, torch.bfloat16)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    losses.append(float(loss))
    print(json.dumps({
        "metric": "RWKV-6 1.6B-shaped training step through the torch binding, tokens/s", "n_gpus": 1,
        "value": B * T / (ms * 1e-3), "unit": "tokens/s", "ms_per_step": ms, "steps": steps, "warmup": warm,
        "config": {"workload": "c4: 24 layers d=2048 H=32 N=64 FFN=7168 vocab=65536, B=8 T=1024, bf16 autocast, AdamW"},
        "parameters": sum(p.numel() for p in model.parameters()),
        "loss_first_last": [losses[0], losses[-1]], "dtype": "bf16", "data": "synthetic"}))


def bench_shift_mix(a):
    """The input side of the time-mix layer at the layer shape of configuration 2 (B=8, T=1024, C=2048,
    mixers of rank 32): the four kernels through the C ABI with pre-allocated buffers, each timed on
    its own with events on torch's current stream.  Prints its own JSON line: microseconds per kernel
    and the rate at which each moves its algorithmic bytes (the (B,T,C) tensors it must read and write)."""
    import torch
    from rwkv_kernel import _native

    lib = _native.load()
    B, T, C, R = 8, 1024, 2048, 32
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(a.seed)
    unit = B * T * C * 2                                   # bytes of one (B,T,C) bf16 tensor
    # all (B,T,C) tensors out of one pool, each base --stagger bytes further on than the one before
    pitch = unit + a.stagger
    pool = torch.empty(22 * pitch, dtype=torch.uint8, device=dev)
    slot = lambda i: pool[i * pitch: i * pitch + unit].view(torch.bfloat16).view(B, T, C)
    fill = lambda i: slot(i).copy_(torch.randn(B, T, C, generator=g).to(torch.bfloat16))
    x, gxm = fill(0), fill(1)
    h = torch.tanh(torch.randn(B, T, 5, R, generator=g)).to(torch.bfloat16).to(dev)
    w2t = (torch.randn(5, C, R, generator=g) / R ** 0.5).to(torch.bfloat16).to(dev)
    bias, mix = torch.rand(5, C, generator=g).to(dev), torch.rand(C, generator=g).to(dev)
    outs, gouts = [slot(2 + i) for i in range(5)], [fill(7 + i) for i in range(5)]
    x_mix, gp, gxx, gx = (slot(12 + i) for i in range(4))
    gcoef, plane = slot(16), pitch // 2                    # five slots in a row
    gmix = torch.empty(C, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()
    calls = {   # name: (call, (B,T,C) tensors read + written)
        "shift_mix_x": (lambda: lib.wkv6_shift_mix_x(st, _native.BF16, B, T, C, P(x), P(mix), P(x_mix)), 2),
        "shift_mix_five": (lambda: lib.wkv6_shift_mix_five(st, _native.BF16, B, T, C, R, P(x), P(h), P(w2t), P(bias),
                                                           *[P(o) for o in outs]), 6),
        "shift_mix_five_backward": (lambda: lib.wkv6_shift_mix_five_backward(
            st, _native.BF16, B, T, C, R, P(x), P(h), P(w2t), P(bias), *[P(o) for o in gouts], P(gcoef), plane, P(gp), P(gxx)), 13),
        "shift_mix_x_backward": (lambda: lib.wkv6_shift_mix_x_backward(st, _native.BF16, B, T, C, P(x), P(mix), P(gp), P(gxx),
                                                                       P(gxm), P(gx), P(gmix)), 5),
    }
    res = {}
    for name, (call, units) in calls.items():
        for _ in range(a.warmup):
            _native.check(call())
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(a.steps):
            call()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / a.steps * 1e3
        res[name] = {"us": us, "algorithmic_bytes": units * unit, "GB/s": units * unit / us * 1e-3,
                     "frac_of_hbm_peak": units * unit / us * 1e-3 / HBM_PEAK_GBS}
    total = sum(v["us"] for v in res.values())
    print(json.dumps({
        "metric": "time-mix input side (token shift + five low-rank mixers), forward + backward kernels, Mtokens/s",
        "n_gpus": 1, "value": B * T / total, "unit": "Mtokens/s", "us_all_four_kernels": total, "steps": a.steps, "warmup": a.warmup,
        "config": {"workload": "mix: B=8 T=1024 C=2048 rank 32, bf16", "allocation": "one pool, tensor bases %d B apart mod 2 MiB" % a.stagger}, "kernels": res, "dtype": "bf16", "data": "synthetic"}))


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build measures ONE GPU; --gpus %d is not supported "
              "(every (batch, head) pair is independent: more GPUs split B or H with no exchange)" % a.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from rwkv_kernel import _native

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    if a.workload == "c5":
        torch.cuda.set_device(0)
        return bench_stateful(a)
    if a.workload == "c4":
        torch.cuda.set_device(0)
        return bench_model_step(a)
    if a.workload == "mix":
        torch.cuda.set_device(0)
        return bench_shift_mix(a)
    lib = _native.load()
    B, T, H, dt_name = WORKLOADS[a.workload]
    N = 64
    C = H * N
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32, "f16": torch.float16}[dt_name]
    odtype = torch.float32 if dt_name == "f16" else dtype   # fp16 tensors: fp32 outputs (and upstream gradient)
    code = {"bf16": _native.BF16, "f32": _native.F32, "f16": _native.F16}[dt_name]
    es = 4 if dt_name == "f32" else 2                       # bytes per input element
    eo = 2 if dt_name == "bf16" else 4                      # bytes per output element
    algo = {"auto": _native.ALGO_AUTO, "scan": _native.ALGO_SCAN, "chunk": _native.ALGO_CHUNK}[a.algo]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # The ten (B,T,C) tensors and the saved states come out of one block, each base `--stagger` bytes
    # further from a 2 MiB boundary than the one before: a workgroup walks all of them row by row in
    # step, and tensors whose bases agree modulo 4 KiB send all those streams to the same memory
    # channel at the same time (which costs about 5 % at this size; torch's own allocator returns
    # 2 MiB-aligned blocks).  The torch flavour carves the tensors it allocates itself the same way.
    nsave = 0 if a.plain_pair else lib.wkv6_saved_bytes(code, algo, B, T, C, H)
    ins = synthetic_inputs(B, T, H, N, a.seed)
    u = ins[4].to(dtype).to(dev).contiguous()
    stream = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()

    def make_calls(stagger):
        nbytes = B * T * C * max(es, eo)
        slot = (nbytes + (2 << 20) - 1) // (2 << 20) * (2 << 20) + (2 << 20)
        pool = torch.empty(11 * slot + nsave + (2 << 20), dtype=torch.uint8, device=dev)
        first = -pool.data_ptr() % (2 << 20)

        def carve(i, nb=nbytes):
            o = first + i * slot + i * stagger
            return pool[o:o + nb]

        def big(i, src=None, dt=None):
            dt = dt or dtype
            t = carve(i, B * T * C * torch.empty((), dtype=dt).element_size()).view(dt).view(B, T, C)
            if src is not None:
                t.copy_(src.to(dt))
            return t

        r, k, v, w = (big(i, ins[i]) for i in range(4))
        gy = big(4, ins[5], odtype)
        y, gr, gk, gv, gw = (big(5 + i, None, odtype) for i in range(5))
        gu_part = torch.empty(B, C, dtype=odtype, device=dev)
        fws_bytes = lib.wkv6_forward_workspace_bytes(code, algo, B, T, C, H)
        bws_bytes = lib.wkv6_backward_workspace_bytes_ex(code, algo, B, T, C, H)
        fws = torch.empty(max(fws_bytes, 16), dtype=torch.uint8, device=dev)
        bws = torch.empty(max(bws_bytes, 16), dtype=torch.uint8, device=dev)

        # the pair a training step uses (the torch autograd.Function does the same): the forward saves the
        # per-chunk states the backward would otherwise recompute; --plain-pair times the two calls the
        # reference's binding corresponds to (forward(r..y), backward(r..gu)) instead
        saved = carve(10, max(nsave, 16))

        def fwd():
            if nsave:
                _native.check(lib.wkv6_forward_save(stream, code, algo, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y),
                                                    P(saved), nsave))
            else:
                _native.check(lib.wkv6_forward_ex(stream, code, algo, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y),
                                                  P(fws), fws_bytes))

        gu_sum = torch.empty(C, dtype=odtype, device=dev)

        def bwd_call():
            if nsave:   # the batch sum of gu comes out of the same launch
                _native.check(lib.wkv6_backward_saved_sum(stream, code, algo, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                                          P(gr), P(gk), P(gv), P(gw), P(gu_part), P(gu_sum), P(saved), nsave))
            else:
                _native.check(lib.wkv6_backward_ex(stream, code, algo, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                                   P(gr), P(gk), P(gv), P(gw), P(gu_part), P(bws), bws_bytes))

        def bwd():   # what a training step does: the library call plus the batch sum of gu, as the reference's binding
            bwd_call()
            return gu_sum if nsave else torch.sum(gu_part, 0)

        def step():
            fwd(); bwd()

        return fwd, bwd_call, bwd, step

    fwd, bwd_call, bwd, step = make_calls(a.stagger)
    preheat_ms = preheat(step, a.preheat_ms) if a.preheat_ms > 0 else 0.0
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        fwd(); bwd()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / a.steps * 1e3
    tokens = B * T

    # Per-launch GPU durations with events on the launch stream (torch's current stream), taken inside
    # the same alternating forward / backward sequence the timed region runs (a kernel launched after
    # itself instead of after its partner finds other data in the 256 MB Infinity Cache and takes a few
    # microseconds longer): event, forward, event, backward, event.
    def gpu_ms_pair(reps):
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(reps)]
        for e0, e1, e2 in ev:
            e0.record(); fwd(); e1.record(); bwd_call(); e2.record()
        torch.cuda.synchronize()
        tf = sorted(e0.elapsed_time(e1) for e0, e1, _ in ev)
        tb = sorted(e1.elapsed_time(e2) for _, e1, e2 in ev)
        return sum(tf) / len(tf), tf[len(tf) // 2], sum(tb) / len(tb), tb[len(tb) // 2]

    def gpu_ms(fn, reps):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for s, e in ev:
            s.record(); fn(); e.record()
        torch.cuda.synchronize()
        ts = sorted(s.elapsed_time(e) for s, e in ev)
        return sum(ts) / len(ts), ts[len(ts) // 2]

    reps = max(10, min(a.steps, 50))
    f_avg, f_med, b_avg, b_med = gpu_ms_pair(reps)   # (the backward: the kernel alone, one launch per call)

    # stream-copy bandwidth actually reachable on this box (read + write of a 1 GiB buffer)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    c_avg, _ = gpu_ms(lambda: dst.copy_(src), 10)
    copy_gbs = 2 * src.numel() / (c_avg * 1e-3) / 1e9
    del src, dst

    bytes_fwd = B * T * C * (4 * es + eo) + C * es                # r, k, v, w in, y out
    bytes_bwd = B * T * C * (4 * es + eo + 4 * eo) + C * (es + eo)   # r, k, v, w, gy in, four gradients out
    bytes_step = bytes_fwd + bytes_bwd
    dom = "bwd" if b_avg >= f_avg else "fwd"
    dom_bytes, dom_ms = (bytes_bwd, b_avg) if dom == "bwd" else (bytes_fwd, f_avg)
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    step_gbs = bytes_step / (ms_per_step * 1e-3) / 1e9
    algo_used = a.algo

    out = {
        "metric": "WKV6 fwd+bwd Mtokens/s + %% HBM roofline, B%d T%d C%d H%d %s" % (B, T, C, H, dt_name),
        "value": tokens / (ms_per_step * 1e-3) / 1e6,
        "unit": "Mtokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "preheat_ms": preheat_ms, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt_name, "data": "synthetic",
        "config": {"workload": "%s: WKV6 fwd+bwd B=%d T=%d C=%d H=%d N=%d %s I/O fp32 state" % (
            a.workload, B, T, C, H, N, dt_name), "algo": algo_used, "tokens_per_step": tokens,
            "calls": "forward+backward" if (a.plain_pair or not nsave) else "forward_save+backward_saved_sum",
            "allocation": "one block, tensor bases staggered by %d B" % a.stagger},
        "roofline": {
            "bound": "hbm", "kernel": "wkv6_%s (%s)" % ("backward" if dom == "bwd" else "forward", algo_used),
            "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": None if a.plain_pair else MEASURED_TRAFFIC_BYTES.get((a.workload, algo_used, dom)),
            "algorithmic_bytes": dom_bytes, "avg_ms": dom_ms,
        },
        "fwd_bwd": {
            "algorithmic_bytes": bytes_step, "achieved_GBps": step_gbs, "frac_of_hbm_peak": step_gbs / HBM_PEAK_GBS,
            "frac_of_measured_copy": step_gbs / copy_gbs, "measured_copy_GBps": copy_gbs,
            "fwd_ms_avg": f_avg, "fwd_ms_median": f_med, "bwd_ms_avg": b_avg, "bwd_ms_median": b_med,
            "fwd_GBps": bytes_fwd / (f_avg * 1e-3) / 1e9, "bwd_GBps": bytes_bwd / (b_avg * 1e-3) / 1e9,
        },
    }
    def timed_ms(fn, steps):
        """GPU time per call of fn over `steps` back-to-back calls (events on the launch stream)."""
        for _ in range(max(30, a.warmup // 5)):   # (the framework's caching allocator settles within the first calls)
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    if a.stagger and not a.plain_pair and not a.no_extra_timings:
        # the same calls on tensors whose bases all sit on 2 MiB boundaries (what a framework's allocator returns)
        out["unstaggered_ms_per_step"] = timed_ms(make_calls(0)[3], a.steps)
    if dt_name == "bf16" and not a.plain_pair and a.algo == "auto" and not a.no_extra_timings:
        # what a caller of the torch binding gets: op(r, k, v, w, u) and y.backward(gy) on tensors from separate
        # torch.empty calls (the binding staggers only what it allocates itself: y, the saved block, the gradients).
        # The binding's host side (autograd bookkeeping, seven allocations per step) is inside this figure.
        from rwkv_kernel import RWKVKernelOperator
        op = RWKVKernelOperator(N, T)
        leaves = []
        for i in range(4):
            t = torch.empty(B, T, C, dtype=dtype, device=dev)
            t.copy_(ins[i].to(dtype))
            leaves.append(t.requires_grad_(True))
        ub = u.clone().requires_grad_(True)
        gyb = torch.empty(B, T, C, dtype=odtype, device=dev)
        gyb.copy_(ins[5].to(odtype))

        def binding_step():
            for t in leaves:
                t.grad = None
            ub.grad = None
            yb, _ = op(*leaves, ub)
            yb.backward(gyb)

        out["binding_ms_per_step"] = timed_ms(binding_step, max(a.steps, 100))   # (host-bound: a short run is noisy)
        # the same step captured once and replayed: the binding's kernels on the binding's own allocation, without its
        # host side (the situation inside a model step, where the host runs ahead of the GPU)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            binding_step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            binding_step()
        out["binding_replayed_ms_per_step"] = timed_ms(graph.replay, a.steps)
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(B, T, H, N, a.seed, a.cpu_tokens)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
