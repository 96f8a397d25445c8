"""Throughput and per-kernel roofline fractions of the Rukedra design (latent attention, minGRU, grouped norms with gated
residual branches, sigmoid-routed experts) beside the closest llama-shaped model of the framework at equal sizes --
``python bench.py --rukedra``.

Model level: prefill tokens/s (whole prompts in one ragged step vs. the padded-grid prefill) and decode tokens/s (one token per
sequence and step; eager and captured) for a few layers at the widths of a small production model, random weights.  Kernel
level: every kernel of the design timed alone (HIP events around a loop of launches) with its algorithmic bytes and flops, next
to the like kernel of the framework's other models at the same shape; ``far`` = how many times further from its roofline (HBM
8 TB/s or 2.5 PFLOP/s dense 16-bit MFMA, whichever bounds it) the new kernel is than its counterpart."""

from __future__ import annotations

import time

import torch

from .layered_bench import _entry, _time


def _step_of(dev, batch, first, count):
    from lite_llama_amd.executor.ragged import RaggedStep

    n = batch * count
    vec = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)   # noqa: E731
    return RaggedStep(num_tokens=n, num_seqs=batch, tok_seq=vec([i for i in range(batch) for _ in range(count)]),
                      tok_pos=vec([first + j for _ in range(batch) for j in range(count)]),
                      select=vec([i * (first + count) + first + j for i in range(batch) for j in range(count)]),
                      seq_start=vec([i * count for i in range(batch + 1)]), seq_first_pos=vec([first] * batch),
                      seq_slot=vec(list(range(batch))), seq_parity=vec([0] * batch), longest_run=count,
                      longest_context=first + count)


def kernel_table(dev, dtype, width, heads, dim, rot, vdim, rank, ff, gru, experts, top, eff, window, prefill=(8, 512), decode=(32, 1024)):
    from lite_llama_amd.kernels import flash_attention2_no_pad, flash_decoding, skip_rmsnorm, swiglu_forward
    from lite_llama_amd.kernels.attention import latent_kv_prep, ragged_attention, rotate_pairs
    from lite_llama_amd.kernels.fused_moe import fused_moe, group_router, moe_route_topk, sparse_glu_experts
    from lite_llama_amd.kernels.norm_act import GatedUpdate, gated_group_norm, glu_act
    from lite_llama_amd.kernels.recurrent import gated_linear_scan, mingru_scan

    es = torch.empty(0, dtype=dtype).element_size()
    h16 = torch.float16 if dtype == torch.float32 else dtype
    out = []
    dk = rank + rot
    hd = dim + rot                                   # the llama path's head width at equal query / key work per head
    for phase, (batch, length) in (("prefill", prefill), ("decode", decode)):
        first, count = (0, length) if phase == "prefill" else (length - 1, 1)
        n = batch * count
        step = _step_of(dev, batch, first, count)
        x = torch.randn(n, width, device=dev)
        y = torch.randn(n, 1, width, device=dev).to(dtype)
        rows = torch.randn(n, 2 * width, device=dev).to(dtype)
        w = torch.ones(width, device=dev, dtype=dtype)
        # post norm + gate + residual add + pre norm vs skip_rmsnorm
        upd = GatedUpdate(y, w, rows[:, width:], w)
        t_new = _time(lambda: gated_group_norm(x, upd, w, 1e-6, 2))
        hx, hr = y.view(n, width).clone(), y.view(n, width).clone()
        t_old = _time(lambda: skip_rmsnorm(hx, hr, w, 1e-6))
        like = _entry("skip_rmsnorm (16-bit residual)", t_old, n * width * es * 4, 0)
        out.append(dict(_entry("gated_group_norm (sum + gate + post norm + fp32 residual + pre norm)", t_new,
                               n * width * (4 + 4 + 3 * es), 0, like), phase=phase))
        # gated activation vs swiglu
        gu = torch.randn(n, 2 * ff + width, device=dev).to(dtype)
        t_new = _time(lambda: glu_act(gu, ff, "gelu_tanh"))
        a, b = torch.randn(n, ff, device=dev).to(h16), torch.randn(n, ff, device=dev).to(h16)
        t_old = _time(lambda: swiglu_forward(a, b))
        like = _entry("swiglu_forward", t_old, n * ff * es * 3, 0)
        out.append(dict(_entry("glu_act (tanh-gelu, column ranges of the fused projection)", t_new, n * ff * es * 3, 0, like), phase=phase))
        # latent rows -> cache, query rotation
        ctx_rows = batch * (first + count)
        cache = torch.randn(ctx_rows, 1, dk, device=dev).to(dtype)
        table = torch.arange(ctx_rows, dtype=torch.int32, device=dev).view(batch, first + count)
        proj = torch.randn(n, dk + 2 * width, device=dev).to(dtype)
        freq = torch.rand(rot // 2, device=dev)
        t_prep = _time(lambda: latent_kv_prep(proj, 0, rank, rot, w[:rank], 1e-6, freq, rot // 2, 1.1, step, cache.view(ctx_rows, dk)))
        q = torch.randn(n, heads, dim + rot, device=dev).to(dtype)
        qa = torch.randn(n, heads, dk, device=dev).to(dtype)
        t_rot = _time(lambda: rotate_pairs(q, dim, rot, freq, rot // 2, 1.1, step, qa, rank))
        out.append(dict(_entry("latent_kv_prep (latent norm + key rotation + cache write)", t_prep, n * dk * es * 2, 0), phase=phase))
        out.append(dict(_entry("rotate_pairs (query heads' rotated part)", t_rot, n * heads * rot * es * 2, 0), phase=phase))
        # attention in the absorbed form vs the llama kernels at the same number of heads
        vc = cache[:, :, :rank]
        for win in (0, window):
            name = f"ragged_attention (absorbed latent, {'window ' + str(win) if win else 'causal'})"
            t_new = _time(lambda: ragged_attention(qa, cache, vc, 0.1, step, table, window=win), iters=5 if phase == "prefill" else 20)
            span = min(win, length) if win else length
            if phase == "prefill":
                pairs = batch * (length * span - span * (span - 1) / 2 if win else length * (length + 1) / 2)
                flops, nbytes = heads * 2.0 * (dk + rank) * pairs, n * (2 * heads * dk + dk) * es
            else:
                flops, nbytes = batch * heads * 2.0 * (dk + rank) * span, batch * span * dk * es
            like = None
            if not win:
                qh = torch.randn(n, heads, 128, device=dev).to(h16)
                kc = torch.randn(ctx_rows, heads, 128, device=dev).to(h16)
                vv = torch.randn(ctx_rows, heads, 128, device=dev).to(h16)
                if phase == "prefill":
                    start = torch.arange(batch, dtype=torch.int32, device=dev) * length
                    lens = torch.full((batch,), length, dtype=torch.int32, device=dev)
                    t_old = _time(lambda: flash_attention2_no_pad(qh, kc, vv, 128 ** -0.5 * 1.4426950408889634, start, lens, length), iters=5)
                    like = _entry("flash_attention2_no_pad (head width 128, one K/V head per query head)", t_old,
                                  n * 4 * heads * 128 * es, batch * heads * 4.0 * 128 * length * length / 2)
                else:
                    req = torch.arange(batch, dtype=torch.int32, device=dev)
                    lens = torch.full((batch,), length, dtype=torch.int32, device=dev)
                    t_old = _time(lambda: flash_decoding(qh, kc, vv, 128 ** -0.5, table, req, lens, length))
                    like = _entry("flash_decoding (head width 128, one K/V head per query head)", t_old,
                                  ctx_rows * 2 * heads * 128 * es, batch * heads * 4.0 * 128 * length)
            out.append(dict(_entry(name, t_new, nbytes, flops, like), phase=phase))
            like_causal = like if not win else like_causal
        if phase == "prefill":   # whole prompts: keys / values expanded per head from the step's own latents (the model's prompt form)
            import dataclasses

            qf = torch.randn(n, heads, dim + rot, device=dev).to(dtype)
            kf = torch.randn(n, heads, dim + rot, device=dev).to(dtype)
            vf = torch.randn(n, heads, vdim, device=dev).to(dtype)
            own = dataclasses.replace(step, seq_slot=torch.arange(batch, dtype=torch.int32, device=dev))
            t_new = _time(lambda: ragged_attention(qf, kf, vf, 0.1, own, table), iters=5)
            pairs = batch * length * (length + 1) / 2
            out.append(dict(_entry("ragged_attention (expanded keys / values, causal: the prompt form of whole prompts)", t_new,
                                   n * heads * (2 * (dim + rot) + 2 * vdim) * es, heads * 2.0 * (dim + rot + vdim) * pairs, like_causal), phase=phase))
        # recurrence vs the framework's other recurrent layer (HGRN2 at the same number of channels)
        zxg = torch.randn(n, 3 * gru + width, device=dev).to(dtype)
        st = torch.zeros(batch, gru, device=dev)
        zb = torch.zeros(gru, device=dev, dtype=dtype)
        t_new = _time(lambda: mingru_scan(zxg, gru, zb, zb, step, st), iters=5 if phase == "prefill" else 20)
        hh, hdv = gru // 128, 128
        qfv = torch.randn(n, 3 * gru, device=dev).to(dtype)
        st2 = torch.zeros(batch, hh, hdv, hdv, device=dev)
        fb = torch.zeros(gru, device=dev, dtype=dtype)
        t_old = _time(lambda: gated_linear_scan(qfv, hh, hdv, hdv, fb, fb, w[:hdv], 1e-6, step, st2), iters=5 if phase == "prefill" else 20)
        like = _entry("gated_linear_scan (HGRN2, heads of 128 x 128)", t_old,
                      n * 4 * gru * es + batch * gru * hdv * 4 * (2 if phase == "decode" else 1), n * gru * hdv * 4.0)
        out.append(dict(_entry("mingru_scan", t_new, n * 4 * gru * es + batch * gru * 4 * 2, n * gru * 12.0, like), phase=phase,
                        note="serial in the tokens of a sequence: one thread per (sequence, channel)"))
        # experts: router, sort + grouped products vs the fp16 softmax-router path of the framework
        h = torch.randn(n, width, device=dev).to(dtype)
        wr = (torch.randn(experts, width, device=dev) * width ** -0.5).to(dtype)
        t_new = _time(lambda: group_router(h, wr, top, 8, 4, 2.5, extra_weight=wr[:1]))
        logits = torch.randn(n, experts, device=dev).to(h16)
        t_old = _time(lambda: moe_route_topk(logits, top))
        like = _entry("moe_route_topk (softmax tail only; its logits come from a library GEMM)", t_old, n * experts * es, 0)
        out.append(dict(_entry("group_router (fp32 logits + sigmoid + groups + top-k + shared scale)", t_new,
                               n * width * es + experts * width * es, n * experts * width * 2.0, like), phase=phase))
        ids, wts, _ = group_router(h, wr, top, 8, 4, 2.5)
        wgu = (torch.randn(experts, 2 * eff, width, device=dev) * width ** -0.5).to(dtype)
        wd = (torch.randn(experts, width, eff, device=dev) * eff ** -0.5).to(dtype)
        t_new = _time(lambda: sparse_glu_experts(h, wgu, wd, ids, wts), iters=5)
        touched = min(experts, n * top)
        flops = n * top * 6.0 * eff * width
        nbytes = touched * 3 * eff * width * es + n * top * (width + 2 * eff + width) * es
        hf, w1, w2 = h.to(torch.float16), wgu.to(torch.float16), wd.to(torch.float16)
        t_old = _time(lambda: fused_moe(hf, w1, w2, wts.to(torch.float16), ids), iters=5)
        like = _entry("fused_moe (fp16: align + two grouped GEMMs + silu + sum)", t_old, nbytes, flops)
        out.append(dict(_entry("sparse_glu_experts (sort + gate|up with silu epilogue + weighted down)", t_new, nbytes, flops, like), phase=phase))
    return out


def _geometry(width, heads, dim, rot, vdim, rank, q_rank, ff, gru, experts, top, eff, shared, window, vocab, layers):
    from lite_llama_amd.model_layers import LayeredGeometry, LayerSpec, MixerSpec, MlpSpec, RotarySpec

    rotary = RotarySpec(rot, 10000.0, 8.0, 4096.0, 32.0, 1.0)
    a1 = MixerSpec("latent_attention", heads=heads, dim=dim, vdim=vdim, scale=(dim + rot) ** -0.5, rot_dim=rot, kv_rank=rank,
                   q_rank=q_rank, window=window, out_gate=True, rotary=rotary)
    a2 = MixerSpec("latent_attention", heads=heads, dim=dim, vdim=vdim, scale=(dim + rot) ** -0.5, rot_dim=rot, kv_rank=rank, rotary=rotary)
    rec = MixerSpec("mingru", width=gru)
    dense = MlpSpec("dense", ff=ff, act="gelu_tanh")
    moe = MlpSpec("moe", ff=eff, act="silu", experts=experts, top=top, group_count=8, group_keep=4, route_scale=2.5, shared_ff=shared)
    cycle = [(a1, dense), (rec, moe), (a2, dense), (rec, moe)]
    specs = tuple(LayerSpec(m, ff=f.ff, mlp_kind=f.kind, mlp=f) for m, f in (cycle[i % 4] for i in range(layers)))
    return LayeredGeometry("rukedra", vocab, width, 1e-6, specs, token_shift=False, sandwich=True, norm_groups=2, logit_softcap=30.0)


def model_points(dev, dtype, geo, llama, prefill=(8, 512), decode=(32, 1024), steps=16):
    from lite_llama_amd.executor import DecodeEngine
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.model import CausalLM, ModelGeometry
    from lite_llama_amd.model_layers import LayeredLM

    vocab = geo.vocab_size
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
    res["rukedra_prefill"] = {"batch": b, "prompt": length, "ms": round(dt * 1e3, 2), "tokens_per_s": round(b * length / dt)}
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
        res["rukedra_decode_captured" if captured else "rukedra_decode"] = {
            "batch": b, "ctx": ctx, "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(b / dt),
            "launches": "one hipGraph per step" if captured else "eager"}
        runner.check_errors()
        del runner
    del model
    torch.cuda.empty_cache()
    # the closest llama-shaped model: same width, heads, feed-forward width and depth; rotary attention + swiglu in every layer
    cgeo = ModelGeometry("bench", llama["width"], len(geo.layers), llama["heads"], llama["heads"], llama["hd"], llama["ff"], vocab)
    h16 = torch.float16 if dtype == torch.float32 else dtype
    cm = CausalLM(cgeo).init_synthetic(0, device=dev).to(h16)
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


SIZES = {
    # widths of a 2B-class model with a compact latent: 16 heads of 64 + 32, latent 192 (one cached row of 224 entries per token)
    "compact": dict(width=2048, heads=16, dim=64, rot=32, vdim=64, rank=192, q_rank=768, ff=5632, gru=2048, experts=32, top=4,
                    eff=704, shared=1408, window=256),
    # a wider model: 24 heads of 96 + 32, latent 224 (rows of 256 entries), more and smaller experts
    "wide": dict(width=3072, heads=24, dim=96, rot=32, vdim=96, rank=224, q_rank=1024, ff=8192, gru=3072, experts=64, top=8,
                 eff=512, shared=1024, window=512),
}


def run(dtype_name="bf16", layers=4, sizes=("compact", "wide"), kernels=True):
    dev = torch.device("cuda", 0)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype_name]
    line = {"metric": "rukedra_throughput", "dtype": dtype_name, "data": "synthetic", "points": {}}
    for name in sizes:
        s = SIZES[name]
        geo = _geometry(vocab=32768, layers=layers, **s)
        llama = dict(width=s["width"], heads=s["heads"], hd=128, ff=s["ff"])
        point = {"sizes": dict(s, layers=layers, vocab=32768), "model": model_points(dev, dtype, geo, llama)}
        if kernels:
            k = {key: s[key] for key in ("width", "heads", "dim", "rot", "vdim", "rank", "ff", "gru", "experts", "top", "eff", "window")}
            point["kernels"] = kernel_table(dev, dtype, **k)
        line["points"][name] = point
        torch.cuda.empty_cache()
    return line
