"""Throughput and per-kernel roofline fractions of the layered family (model_layers.py) beside the closest llama-shaped model
of the framework at equal sizes -- ``python bench.py --layered``.

Model level: prefill tokens/s (whole prompts in one ragged step vs. the padded-grid prefill) and decode tokens/s (one token per
sequence and step, eager launches vs. the llama model's captured step), a few layers at the widths of a 1.5B-class model,
random weights.  Kernel level: every kernel of the new family timed alone (HIP events around a loop of launches) with its
algorithmic bytes and flops, next to the like kernel of the llama path at the same shape; ``far`` = how many times further from
its roofline (HBM 8 TB/s or 2.5 PFLOP/s dense 16-bit MFMA, whichever bounds it) the new kernel is than its counterpart."""

from __future__ import annotations

import time

import torch

HBM, MFMA = 8.0e12, 2.5e15


def _time(fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def _frac(seconds, nbytes, flops):
    bound = max(nbytes / HBM, flops / MFMA)
    return bound / seconds


def _entry(name, seconds, nbytes, flops, like=None):
    e = {"kernel": name, "us": round(seconds * 1e6, 1), "MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 2),
         "roofline_frac": round(_frac(seconds, nbytes, flops), 4)}
    if like is not None:
        e["like"] = like
        e["far"] = round(like["roofline_frac"] / max(e["roofline_frac"], 1e-9), 2)
    return e


def kernel_table(dev, dtype, width, heads, kv_heads, hd, ff, prefill=(8, 512), decode=(32, 1024)):
    from lite_llama_amd.executor.ragged import RaggedStep
    from lite_llama_amd.kernels import flash_attention2_no_pad, flash_decoding, skip_rmsnorm, swiglu_forward
    from lite_llama_amd.kernels.activations import xielu
    from lite_llama_amd.kernels.attention import qk_norm_cache, ragged_attention
    from lite_llama_amd.kernels.norm_act import add_rmsnorm_shift
    from lite_llama_amd.kernels.recurrent import gated_linear_scan

    es = torch.empty(0, dtype=dtype).element_size()
    out = []

    def step_of(batch, first, count):
        n = batch * count
        vec = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        return RaggedStep(num_tokens=n, num_seqs=batch, tok_seq=vec([i for i in range(batch) for _ in range(count)]),
                          tok_pos=vec([first + j for _ in range(batch) for j in range(count)]),
                          select=vec([i * (first + count) + first + j for i in range(batch) for j in range(count)]),
                          seq_start=vec([i * count for i in range(batch + 1)]), seq_first_pos=vec([first] * batch),
                          seq_slot=vec(list(range(batch))), seq_parity=vec([0] * batch), longest_run=count,
                          longest_context=first + count)

    for phase, (batch, length) in (("prefill", prefill), ("decode", decode)):
        first, count = (0, length) if phase == "prefill" else (length - 1, 1)
        n = batch * count
        step = step_of(batch, first, count)
        x = torch.randn(n, width, device=dev)
        delta = torch.randn(n, width, device=dev).to(dtype)
        w = torch.ones(width, device=dev, dtype=dtype)
        state = torch.zeros(2, batch, width, device=dev)
        # norm (+ residual add + shift) vs skip_rmsnorm
        xo = torch.empty_like(x)
        t_new = _time(lambda: add_rmsnorm_shift(x, delta, w, 1e-6, x_out=xo, shift=w, step=step, state=state))
        hx, hr = delta.clone(), delta.clone()
        t_old = _time(lambda: skip_rmsnorm(hx, hr, w, 1e-6))
        like = _entry("skip_rmsnorm (16-bit residual)", t_old, n * width * es * 4, 0)
        out.append(dict(_entry("add_rmsnorm_shift (fp32 residual + token shift)", t_new, n * width * (4 + es + 4 + es), 0, like), phase=phase))
        # activation vs swiglu
        z = torch.randn(n, ff, device=dev).to(dtype)
        pq = torch.tensor([0.3, -0.2], device=dev).to(dtype)
        t_new = _time(lambda: xielu(z, pq))
        z2 = torch.randn(n, ff, device=dev).to(dtype)
        t_old = _time(lambda: swiglu_forward(z, z2))
        like = _entry("swiglu_forward", t_old, n * ff * es * 3, 0)
        out.append(dict(_entry("xielu", t_new, n * ff * es * 2, 0, like), phase=phase))
        # attention
        rows = batch * (first + count)
        kc = torch.randn(rows, kv_heads, hd, device=dev).to(dtype)
        vc = torch.randn(rows, kv_heads, hd, device=dev).to(dtype)
        table = torch.arange(rows, dtype=torch.int32, device=dev).view(batch, first + count)
        qkv = torch.randn(n, (heads + 2 * kv_heads) * hd, device=dev).to(dtype)
        t_prep = _time(lambda: qk_norm_cache(qkv, heads, kv_heads, hd, hd, w[:hd], w[:hd], 1e-6, 0.3, 128, step, kc, vc))
        out.append(dict(_entry("qk_norm_cache (q/k norm + temperature + cache write)", t_prep, n * (heads + 2 * kv_heads) * hd * es * 2, 0),
                        phase=phase))
        q = torch.randn(n, heads, hd, device=dev).to(dtype)
        sink = torch.zeros(heads, device=dev, dtype=dtype)
        t_new = _time(lambda: ragged_attention(q, kc, vc, hd ** -0.5, step, table, sink=sink), iters=5 if phase == "prefill" else 20)
        if phase == "prefill":
            flops = batch * heads * 4.0 * hd * length * length / 2
            nbytes = n * (2 * heads + 2 * kv_heads) * hd * es
            h16 = torch.float16 if dtype == torch.float32 else dtype
            q16, k16, v16 = q.to(h16), kc.to(h16), vc.to(h16)
            start = torch.arange(batch, dtype=torch.int32, device=dev) * length
            lens = torch.full((batch,), length, dtype=torch.int32, device=dev)
            t_old = _time(lambda: flash_attention2_no_pad(q16, k16, v16, hd ** -0.5 * 1.4426950408889634, start, lens, length), iters=5)
            like = _entry("flash_attention2_no_pad", t_old, nbytes, flops)
        else:
            flops = batch * heads * 4.0 * hd * length
            nbytes = rows * 2 * kv_heads * hd * es
            h16 = torch.float16 if dtype == torch.float32 else dtype
            q16, k16, v16 = q.to(h16), kc.to(h16), vc.to(h16)
            req = torch.arange(batch, dtype=torch.int32, device=dev)
            lens = torch.full((batch,), length, dtype=torch.int32, device=dev)
            t_old = _time(lambda: flash_decoding(q16, k16, v16, hd ** -0.5, table, req, lens, length))
            like = _entry("flash_decoding", t_old, nbytes, flops)
        out.append(dict(_entry("ragged_attention (sink, paged)", t_new, nbytes, flops, like), phase=phase))
        # recurrence: no counterpart in the llama path; its own bounds: state traffic (decode), projection rows (prefill)
        qfv = torch.randn(n, 3 * heads * hd, device=dev).to(dtype)
        st = torch.zeros(batch, heads, hd, hd, device=dev)
        fb = torch.zeros(heads * hd, device=dev, dtype=dtype)
        t_new = _time(lambda: gated_linear_scan(qfv, heads, hd, hd, fb, fb, w[:hd], 1e-6, step, st), iters=5 if phase == "prefill" else 20)
        nbytes = n * 4 * heads * hd * es + batch * heads * hd * hd * 4 * (2 if phase == "decode" else 1)
        out.append(dict(_entry("gated_linear_scan (HGRN2)", t_new, nbytes, n * heads * hd * hd * 4.0), phase=phase,
                        note="serial in the tokens of a sequence: batch x heads workgroups"))
    return out


def model_points(dev, dtype, width, heads, kv_heads, hd, ff, vocab, layers, prefill=(8, 512), decode=(32, 1024), steps=16):
    from lite_llama_amd.executor import DecodeEngine
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.model import CausalLM, ModelGeometry
    from lite_llama_amd.model_layers import LayeredGeometry, LayeredLM, LayerSpec, MixerSpec

    att = MixerSpec("attention", heads, hd, hd, kv_heads=kv_heads, scale=hd ** -0.5, temp_coef=0.3, temp_every=128)
    rec = MixerSpec("hgrn2", heads, hd, hd)
    geo = LayeredGeometry("bench", vocab, width, 1e-6, tuple(LayerSpec(att if i % 2 else rec, ff=ff) for i in range(layers)))
    model = LayeredLM(geo, dtype=dtype).init_synthetic(0, dev)
    res = {}
    g = torch.Generator().manual_seed(5)
    b, length = prefill
    runner = RaggedRunner(model, b * (length + 64), b, 64, dev)
    prompts = [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(b)]

    def run_prefill():
        slots = [runner.admit() for _ in range(b)]
        runner.step(list(zip(slots, prompts)))
        torch.cuda.synchronize()
        runner.release(slots)

    run_prefill()
    t0 = time.perf_counter()
    for _ in range(3):
        run_prefill()
    dt = (time.perf_counter() - t0) / 3
    res["layered_prefill"] = {"batch": b, "prompt": length, "ms": round(dt * 1e3, 2), "tokens_per_s": round(b * length / dt)}
    del runner
    b, ctx = decode
    for captured in (False, True):
        runner = RaggedRunner(model, b * (ctx + 64), b, 64, dev, capture_decode=captured)
        slots = [runner.admit() for _ in range(b)]
        for lo in range(0, ctx, 256):
            runner.step([(s, torch.randint(0, vocab, (min(256, ctx - lo),), generator=g).tolist()) for s in slots], [])
        toks = [[1]] * b
        for _ in range(3):
            runner.step(list(zip(slots, toks)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            runner.step(list(zip(slots, toks)))
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        res["layered_decode_captured" if captured else "layered_decode"] = {
            "batch": b, "ctx": ctx, "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(b / dt),
            "launches": ("one hipGraph per step (one small host-to-device copy of the step's vectors in front)" if captured
                         else "eager (host builds the step's vectors every step)")}
        if captured:
            res["layered_decode_captured"]["replays"] = runner.replays
        del runner
    del model
    torch.cuda.empty_cache()
    # the closest llama-shaped model: same widths, rotary attention + swiglu MLP in every layer
    cgeo = ModelGeometry("bench", width, layers, heads, kv_heads, hd, ff, vocab)
    cm = CausalLM(cgeo).init_synthetic(0, device=dev)
    h16 = torch.float16 if dtype == torch.float32 else dtype
    cm = cm.to(h16)
    b, length = prefill
    eng = DecodeEngine(cm, max_batch=b, max_seq_len=length + 8, device=dev, kv_dtype=h16)
    ids = torch.randint(0, vocab, (b, length), generator=g).to(dev)
    eng.prefill(ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        eng.prefill(ids)
        torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / 3
    res["llama_prefill"] = {"batch": b, "prompt": length, "ms": round(dt * 1e3, 2), "tokens_per_s": round(b * length / dt)}
    del eng
    b, ctx = decode
    eng = DecodeEngine(cm, max_batch=b, max_seq_len=ctx + steps + 8, device=dev, kv_dtype=h16)
    first = eng.synthetic_context(b, ctx)
    stamps = []
    eng.decode(first, steps + 4, use_graph=True, on_step=lambda i: (torch.cuda.synchronize(), stamps.append(time.perf_counter())))
    torch.cuda.synchronize()
    dt = (time.perf_counter() - stamps[4]) / steps
    res["llama_decode"] = {"batch": b, "ctx": ctx, "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(b / dt),
                           "launches": "one hipGraph per step"}
    return res


def run(dtype_name="bf16", layers=4):
    dev = torch.device("cuda", 0)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype_name]
    sizes = dict(width=1536, heads=12, kv_heads=2, hd=128, ff=8960)
    line = {"metric": "layered_family_throughput", "dtype": dtype_name, "data": "synthetic", "sizes": dict(sizes, layers=layers, vocab=32768),
            "model": model_points(dev, dtype, vocab=32768, layers=layers, **sizes),
            "kernels": kernel_table(dev, dtype, **sizes)}
    return line
