"""The layered family on the GPU against the plain CPU restatement (oracle/layered.py): each mechanism's kernels alone,
then whole models built from small random checkpoints through the loader, the ragged runner, the paged state cache, the
generation engine and the command line.  float32 runs are held to rounding error; bfloat16 runs to the rounding of their
activations.  No configuration here is the size of a published checkpoint."""

import json
import math
import os
import subprocess
import sys

import pytest
import torch

from tests import _layered as T

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64


def _step(seqs, table=None):
    """RaggedStep from ``(slot, first_pos, count, parity)`` per sequence; ``table [slots, positions]`` names cache rows."""
    from lite_llama_amd.executor.ragged import RaggedStep

    starts, tok_seq, tok_pos, select = [0], [], [], []
    for i, (slot, first, count, _) in enumerate(seqs):
        starts.append(starts[-1] + count)
        tok_seq += [i] * count
        tok_pos += range(first, first + count)
        select += [int(table[slot, p]) if table is not None else 0 for p in range(first, first + count)]

    def vec(v):
        return torch.tensor(v, dtype=torch.int32, device=DEV)

    return RaggedStep(num_tokens=starts[-1], num_seqs=len(seqs), tok_seq=vec(tok_seq), tok_pos=vec(tok_pos), select=vec(select),
                      seq_start=vec(starts), seq_first_pos=vec([s[1] for s in seqs]), seq_slot=vec([s[0] for s in seqs]),
                      seq_parity=vec([s[3] for s in seqs]), longest_run=max(s[2] for s in seqs),
                      longest_context=max(s[1] + s[2] for s in seqs))


def _close(got, want, tol):
    got, want = got.detach().cpu().to(F64), want.to(F64)
    err = (got - want).abs().max().item()
    ref = max(want.abs().max().item(), 1e-6)
    assert err <= tol * ref, f"max error {err:.3e} against a scale of {ref:.3e} (allowed {tol:.1e} of it)"


TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


# ------------------------------------------------------------------------------------------------------------------- #
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 70, 600])   # (70: not a multiple of 4 -> the plain, strided form)
def test_add_norm_shift_reads_previous_rows_state_slots_and_zeros(dtype, width):
    from lite_llama_amd.kernels.norm_act import add_rmsnorm_shift
    from oracle import layered as O

    torch.manual_seed(width)
    seqs = [(2, 0, 5, 0), (0, 7, 1, 1), (3, 3, 2, 0)]           # starts a sequence / one decoded token / a portion inside
    n = sum(s[2] for s in seqs)
    x = torch.randn(n, width, device=DEV)
    delta = torch.randn(n, width, device=DEV).to(dtype)
    w = (1 + 0.1 * torch.randn(width, device=DEV)).to(dtype)
    mu = torch.rand(width, device=DEV).to(dtype)
    state = torch.randn(2, 4, width, device=DEV)
    before = state.clone()
    y, res = add_rmsnorm_shift(x, delta, w, 1e-5, shift=mu, step=_step(seqs), state=state)
    s = x.cpu().to(F64) + delta.cpu().to(F64)
    _close(res, s, 1e-6)
    at, want_state = 0, before.cpu().to(F64)
    for slot, first, count, parity in seqs:
        h = O.rms_norm(s[at:at + count], w.cpu().to(F64), 1e-5)
        prev = torch.zeros_like(h)
        prev[1:] = h[:-1]
        if first > 0:
            prev[0] = before[parity, slot].cpu().to(F64)
        _close(y[at:at + count], h + (prev - h) * mu.cpu().to(F64), TOL[dtype])
        want_state[1 - parity, slot] = h[-1]
        at += count
    _close(state, want_state, 1e-5)                                # the read halves and foreign slots are untouched
    # without a shift: plain add + norm, in place on the residual
    x2 = x.clone()
    y2, res2 = add_rmsnorm_shift(x2, delta, w, 1e-5, x_out=x2)
    assert res2.data_ptr() == x2.data_ptr()
    _close(x2, s, 1e-6)
    _close(y2, O.rms_norm(s, w.cpu().to(F64), 1e-5), TOL[dtype])
    with pytest.raises(ValueError):
        add_rmsnorm_shift(x2, delta, w, 1e-5, x_out=x2, shift=mu, step=_step(seqs), state=state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_xielu_cast_pair_residual_set(dtype):
    from lite_llama_amd.kernels.activations import xielu
    from lite_llama_amd.kernels.norm_act import cast_pair, residual_set
    from oracle import layered as O

    z = torch.linspace(-9, 7, 1003, device=DEV).to(dtype)
    for p, q in ((0.3, -0.8), (-2.0, 1.5), (25.0, 0.0)):
        pq = torch.tensor([p, q], device=DEV).to(dtype)
        _close(xielu(z, pq), O.xielu(z.cpu().to(F64), pq[0].cpu().to(F64), pq[1].cpu().to(F64)), TOL[dtype])
    a, b = torch.randn(7, 33, device=DEV), torch.randn(7, 33, device=DEV)
    d = torch.randn(7, 33, device=DEV).to(dtype)
    _close(cast_pair(a, b, dtype, a_delta=d), torch.cat([a.cpu().to(F64) + d.cpu().to(F64), b.cpu().to(F64)], -1), TOL[dtype])
    _close(cast_pair(a, b, dtype), torch.cat([a, b], -1).cpu(), TOL[dtype])
    bias = torch.randn(33, device=DEV).to(dtype)
    out = residual_set(d, bias)
    assert out.dtype == torch.float32
    _close(out, d.cpu().to(F64) + bias.cpu().to(F64), 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dk,dv", [(2, 24, 16), (1, 8, 40), (3, 16, 96), (1, 130, 7), (2, 64, 128), (1, 128, 256)])
def test_gated_linear_scan_carries_state_across_steps_and_ignores_stale_slots(dtype, heads, dk, dv):
    from lite_llama_amd.kernels.recurrent import gated_linear_scan
    from oracle import layered as O

    torch.manual_seed(dk * dv)
    width, eps = 32, 1e-5
    wq, wf, wv = (torch.randn(heads * dk, width) * 0.3, torch.randn(heads * dk, width) * 0.3, torch.randn(heads * dv, width) * 0.3)
    fb, lower = torch.randn(heads * dk).to(dtype), (torch.rand(heads * dk) * 0.95).to(dtype)
    nw = (1 + 0.1 * torch.randn(dv)).to(dtype)
    lens = {1: 12, 0: 12}                                       # slot -> sequence length
    hs = {s: torch.randn(n, width) for s, n in lens.items()}
    rows = {s: (h @ torch.cat([wq, wf, wv]).T).to(dtype) for s, h in hs.items()}   # the fused projection's output
    want = {s: O.hgrn2(hs[s].to(F64), *[t.to(F64) for t in (wq, wf)], fb.to(F64), lower.to(F64), wv.to(F64), nw.to(F64),
                       torch.eye(heads * dv, dtype=F64), heads, dk, dv, eps) for s in lens}
    if dtype != torch.float32:                                   # the oracle must see the rounded projection rows
        def from_rows(r):
            r = r.to(F64)
            q = torch.nn.functional.silu(r[:, :heads * dk]).view(-1, heads, dk)
            f = (lower.to(F64) + (1 - lower.to(F64)) * torch.sigmoid(r[:, heads * dk:2 * heads * dk] + fb.to(F64))).view(-1, heads, dk)
            v = r[:, 2 * heads * dk:].view(-1, heads, dv)
            S, out = torch.zeros(heads, dk, dv, dtype=F64), []
            for t in range(r.shape[0]):
                S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
                out.append(torch.einsum("hkv,hk->hv", S, q[t]))
            return O.rms_norm(torch.stack(out), nw.to(F64), eps).reshape(r.shape[0], -1)
        want = {s: from_rows(rows[s]) for s in lens}
    state = torch.full((3, heads, dk, dv), 7.0, device=DEV)      # garbage an earlier owner of the slots left
    got = {s: [] for s in lens}
    plan = [[(1, 0, 11), (0, 0, 3)], [(1, 11, 1), (0, 3, 9)]]    # portions, then a decoded token beside a portion
    for step_seqs in plan:
        step = _step([(s, f, c, 0) for s, f, c in step_seqs])
        qfv = torch.cat([rows[s][f:f + c] for s, f, c in step_seqs]).to(DEV).contiguous()
        out = gated_linear_scan(qfv, heads, dk, dv, fb.to(DEV), lower.to(DEV), nw.to(DEV), eps, step, state)
        at = 0
        for s, f, c in step_seqs:
            got[s].append(out[at:at + c])
            at += c
    for s in lens:
        _close(torch.cat(got[s]), want[s], 5e-5 if dtype == torch.float32 else 2e-2)
    assert torch.all(state[2] == 7.0)                             # a slot nobody rode is untouched


def _attention_case(dtype, heads, kv_heads, dk, dv, T_len, plan, temp=(0.4, 5), scale=None, qkv_rows=None, sink=None):
    """Runs qk_norm_cache + ragged_attention over ``plan`` (steps of (slot, first, count)) for ONE sequence in slot 1 next to
    a distractor in slot 0; returns (got [T, heads dv], oracle [T, heads dv])."""
    from lite_llama_amd.kernels.attention import qk_norm_cache, ragged_attention
    from oracle import layered as O

    g = torch.Generator().manual_seed(dk * 131 + dv)
    width = (heads + kv_heads) * dk + kv_heads * dv
    rows = qkv_rows if qkv_rows is not None else torch.randn(T_len, width, generator=g)
    rows = rows.to(dtype)
    other = torch.randn(T_len, width, generator=g).to(dtype)
    qn, kn = (1.5 + 0.2 * torch.randn(dk, generator=g)).to(dtype), (1.5 + 0.2 * torch.randn(dk, generator=g)).to(dtype)
    sink = (torch.randn(heads, generator=g) if sink is None else sink).to(dtype)
    scale = scale if scale is not None else dk ** -0.5
    eye = torch.eye(width, dtype=F64)
    q_end, k_end = heads * dk, (heads + kv_heads) * dk
    want = O.sink_attention(rows.to(F64), eye[:q_end], eye[q_end:k_end], eye[k_end:], qn.to(F64), kn.to(F64), sink.to(F64),
                            torch.eye(heads * dv, dtype=F64), heads, kv_heads, dk, dv, scale, temp[0], temp[1], 1e-5)
    pool = 2 * T_len + 5
    perm = torch.randperm(pool, generator=g)[: 2 * T_len].view(2, T_len).to(torch.int32)   # cache rows in no order at all
    table = perm.to(DEV)
    kc = torch.full((pool, kv_heads, dk), float("nan"), device=DEV, dtype=dtype)
    vc = torch.full((pool, kv_heads, dv), float("nan"), device=DEV, dtype=dtype)
    got = []
    for seqs in plan:
        step = _step([(s, f, c, 0) for s, f, c in seqs], table=perm)
        qkv = torch.cat([(rows if s == 1 else other)[f:f + c] for s, f, c in seqs]).to(DEV).contiguous()
        q = qk_norm_cache(qkv, heads, kv_heads, dk, dv, qn.to(DEV), kn.to(DEV), 1e-5, temp[0], temp[1], step, kc, vc)
        out = ragged_attention(q, kc, vc, scale, step, table, sink=sink.to(DEV))
        at = 0
        for s, f, c in seqs:
            if s == 1:
                got.append(out[at:at + c])
            at += c
    return torch.cat(got), want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dk,dv", [(6, 2, 40, 24), (2, 2, 64, 96), (3, 1, 12, 160), (1, 1, 8, 8)])
def test_sink_attention_portions_decode_and_a_neighbour_in_the_batch(dtype, heads, kv_heads, dk, dv):
    plan = [[(1, 0, 33), (0, 0, 2)], [(0, 2, 40), (1, 33, 2)], [(1, 35, 35)]] + [[(0, 42 + i, 1), (1, 70 + i, 1)] for i in range(5)]
    got, want = _attention_case(dtype, heads, kv_heads, dk, dv, 75, plan)
    _close(got, want, 5e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("far", [0, 3, 63, 64, 127, 128, 255, 256, 600])
def test_one_far_key_among_hundreds_is_found(far, dtype):
    """Query and key of one far position are made parallel and the scale sharp: the output must be that position's value,
    from a prompt portion and from a decoded token alike."""
    heads, kv_heads, dk, dv, T_len = 2, 1, 16, 8, 700
    g = torch.Generator().manual_seed(far)
    rows = torch.randn(T_len, (heads + kv_heads) * dk + kv_heads * dv, generator=g)
    u = torch.randn(dk, generator=g)
    rows[far, heads * dk:(heads + 1) * dk] = u                    # the far key ...
    for t in (T_len - 1, T_len - 2):
        rows[t, :dk] = u                                          # ... is what head 0 of the last two tokens asks for
    plan = [[(1, 0, 64)], [(1, 64, T_len - 65)], [(1, T_len - 1, 1)]]   # the last token is decoded alone
    ones = torch.ones(dk)
    sink = torch.tensor([-30.0, 0.5])
    sharp = 4.0 if dtype == torch.float32 else 1.0   # (16-bit queries and keys: a score of 36 +- 0.1 instead of 144 +- 0.5)
    got, want = _attention_case(dtype, heads, kv_heads, dk, dv, T_len, plan, temp=(0.0, 1), scale=sharp, qkv_rows=rows, sink=sink)
    _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)
    v_far = rows[far, (heads + kv_heads) * dk:].to(dtype)
    for t in (T_len - 1, T_len - 2):
        _close(got[t, :dv], v_far.float(), 1e-3 if dtype == torch.float32 else 1e-2)


def test_sink_takes_its_share_of_the_softmax():
    """A sink far above every score leaves nothing for the values; one far below changes nothing; position 0 sees only
    itself and the sink."""
    heads, kv_heads, dk, dv = 2, 2, 16, 8
    plan = [[(1, 0, 20)]]
    hi, want_hi = _attention_case(torch.float32, heads, kv_heads, dk, dv, 20, plan, sink=torch.tensor([40.0, -40.0]))
    _close(hi, want_hi, 5e-5)
    assert hi[:, :dv].abs().max().item() < 1e-6 and hi[:, dv:].abs().max().item() > 1e-2
    mid, want_mid = _attention_case(torch.float32, heads, kv_heads, dk, dv, 20, plan, sink=torch.tensor([0.0, 0.0]))
    _close(mid, want_mid, 5e-5)
    assert (mid[0].abs() < want_hi[0, dv:].abs().max() + 10).all() and not torch.allclose(mid[:, dv:].cpu(), hi[:, dv:].cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dk,dv", [(20, 1, 32, 16), (4, 2, 128, 128), (2, 1, 200, 72)])
def test_decoded_tokens_over_several_partitions_of_the_context(dtype, heads, kv_heads, dk, dv):
    """Contexts of 250 .. 530 tokens: decoded tokens see one, two and three partitions (cut every 256 keys), a group of 20
    query heads needs two column tiles; a neighbour with a short context rides along."""
    T_len = 530
    plan = [[(1, 0, 250), (0, 0, 3)]] + [[(1, 250 + i, 1), (0, 3 + i, 1)] for i in range(10)] + [[(1, 260, 250)]] + \
           [[(1, 510 + i, 1), (0, 13 + i, 1)] for i in range(20)]
    got, want = _attention_case(dtype, heads, kv_heads, dk, dv, T_len, plan, temp=(0.3, 128))
    _close(got, want, 5e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("every", [1, 3, 64])
def test_query_temperature_steps_at_its_period(every):
    """Positions every - 2 .. every + 1 straddle the first step of floor((p + 1) / every)."""
    n = max(2 * every + 2, 8)
    plan = [[(1, 0, n - 3)]] + [[(1, n - 3 + i, 1)] for i in range(3)]
    got, want = _attention_case(torch.float32, 2, 1, 16, 8, n, plan, temp=(0.9, every), scale=1.0)
    _close(got, want, 5e-5)


# ------------------------------------------------------------------------------------------------------------------- #
# whole models through loader, runner and cache
# ------------------------------------------------------------------------------------------------------------------- #
_MODELS = {}


def _model(tmp_path_factory, name, dtype):
    from lite_llama_amd.weights import load_pretrained

    key = (name, dtype)
    if key not in _MODELS:
        cfg = T.CONFIGS[name]
        tens = T.tensors(cfg, seed=len(name))
        folder = T.write(tmp_path_factory.mktemp(name), cfg, tens)
        _MODELS[key] = (load_pretrained(folder, device=DEV, dtype=dtype), cfg, tens, folder)
    return _MODELS[key]


def _feed(runner, slot, tokens, sizes):
    """Feeds ``tokens`` in portions of the given sizes (the last size repeats); returns all logits ``[T, vocab]``."""
    at, out, k = 0, [], 0
    while at < len(tokens):
        c = min(sizes[min(k, len(sizes) - 1)], len(tokens) - at)
        out.append(runner.step([(slot, tokens[at:at + c])], list(range(c))))
        at, k = at + c, k + 1
    return torch.cat(out)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_whole_prompt_layers_and_logits(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import layered as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = T.prompt(cfg, 45)
    want, layers = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 64, 2, block_size=16, device=DEV)
    got_layers = []
    got = runner.step([(runner.admit(), toks)], list(range(len(toks))), collect_layers=got_layers)
    runner.check_errors()
    for i, layer in enumerate(got_layers):
        _close(layer, layers[i], 2e-5)
    _close(got, want, 2e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
@pytest.mark.parametrize("sizes", [[1], [2], [3, 2, 7, 1, 16, 5], [40, 1]])
def test_portions_and_token_by_token_decoding_equal_the_whole_prompt(tmp_path_factory, name, sizes):
    """Portions down to two tokens, pure token-by-token decoding from the first token on, and a long portion followed by
    decoding; pages of 8 tokens, so portions start and end inside pages."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import layered as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = T.prompt(cfg, 58, seed=1)
    want, _ = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 64, 2, block_size=8, device=DEV)
    _close(_feed(runner, runner.admit(), toks, sizes), want, 2e-5)
    runner.check_errors()


def test_unequal_requests_in_one_batch_equal_each_alone_and_freed_pages_and_slots_are_used_again(tmp_path_factory):
    """Four requests of different lengths ride together in changing portions, three slots and a pool that only holds them
    because finished requests give their pages back; a late request takes over a used slot and used pages."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import layered as O

    model, cfg, tens, _ = _model(tmp_path_factory, "loop0", torch.float32)
    lens = {"a": 41, "b": 9, "c": 26, "d": 33}
    toks = {k: T.prompt(cfg, n, seed=ord(k)) for k, n in lens.items()}
    want = {k: O.forward(cfg, tens, v)[0] for k, v in toks.items()}
    runner = RaggedRunner(model, 96, 3, block_size=8, device=DEV)      # 12 pages: a + b + c need 11, d needs 5
    sizes = {"a": [5, 1, 1, 9, 2, 30], "b": [2, 1, 3, 1, 1, 1], "c": [1, 13, 2, 2, 8], "d": [16, 1, 1, 15]}
    at, slot, got, k = {x: 0 for x in lens}, {}, {x: [] for x in lens}, 0
    waiting, live = ["a", "b", "c", "d"], []
    while waiting or live:
        while waiting and runner.free_slots and runner.blocks_held() + runner.blocks_for(lens[waiting[0]]) <= runner.total_blocks:
            name = waiting.pop(0)
            slot[name] = runner.admit()
            live.append(name)
        entries, rows, owners, base = [], [], [], 0
        for name in live:
            if (k + ord(name)) % 4 == 0 and len(live) > 1:
                continue                                              # left out of this step, goes on later
            c = min(sizes[name][min(k, len(sizes[name]) - 1)], lens[name] - at[name])
            entries.append((slot[name], toks[name][at[name]:at[name] + c]))
            rows += range(base, base + c)
            owners += [name] * c
            base, at[name] = base + c, at[name] + c
        k += 1
        if not entries:
            continue
        out = runner.step(entries, rows)
        for j, name in enumerate(owners):
            got[name].append(out[j:j + 1])
        ended = [n for n in live if at[n] == lens[n]]
        runner.release([slot[n] for n in ended])
        live = [n for n in live if n not in ended]
    runner.check_errors()
    assert slot["d"] in (slot["a"], slot["b"], slot["c"])               # d rode a slot somebody had used before
    assert runner.cache.free_blocks == runner.total_blocks
    for name in lens:
        _close(torch.cat(got[name]), want[name], 2e-5)


def test_long_decoding_over_many_pages(tmp_path_factory):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import layered as O

    model, cfg, tens, _ = _model(tmp_path_factory, "once", torch.float32)
    toks = T.prompt(cfg, 150, seed=5)
    want, _ = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 160, 1, block_size=16, device=DEV)
    _close(_feed(runner, runner.admit(), toks, [6, 1]), want, 3e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_bfloat16_model_tracks_the_oracle_and_its_own_portions(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import layered as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.bfloat16)
    toks = T.prompt(cfg, 70, seed=2)
    want, _ = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 160, 2, block_size=16, device=DEV)
    whole = _feed(runner, runner.admit(), toks, [70]).float().cpu()
    parts = _feed(runner, runner.admit(), toks, [2, 9, 1, 1, 30, 1]).float().cpu()
    spread = want.std().item()
    assert (whole.to(F64) - want).pow(2).mean().sqrt().item() < 0.06 * spread
    assert (parts - whole).pow(2).mean().sqrt().item() < 0.03 * spread      # same rounding points, other GEMM shapes


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_replay_like_eager_ones(tmp_path_factory, dtype):
    """Decode-only steps from a hipGraph per (running set, context partitions) cell against the same steps launched eagerly:
    many replays with eager work between them (a neighbour's prompt portions change the running set and come back), a context
    that grows across a partition edge (a second cell for the same slots), every replay compared."""
    from lite_llama_amd.executor.ragged import RaggedRunner

    model, cfg, _, _ = _model(tmp_path_factory, "loop0", dtype)
    a, b = T.prompt(cfg, 290, seed=21), T.prompt(cfg, 40, seed=22)
    eager = RaggedRunner(model, 512, 2, block_size=16, device=DEV)
    graph = RaggedRunner(model, 512, 2, block_size=16, device=DEV, capture_decode=True)
    out = {"eager": [], "graph": []}
    for name, r in (("eager", eager), ("graph", graph)):
        sa, sb = r.admit(), r.admit()
        r.step([(sa, a[:240])], [])
        for i in range(240, 262):                                   # one sequence decoding: 256 is a partition edge
            out[name].append(r.step([(sa, a[i:i + 1])]).float().cpu().clone())
        r.step([(sa, a[262:263]), (sb, b[:30])], [])                 # a mixed step in between (eager in both runners)
        for i in range(10):                                         # two sequences decoding together
            out[name].append(r.step([(sa, a[263 + i:264 + i]), (sb, b[30 + i:31 + i])]).float().cpu().clone())
        r.release([sb])
        for i in range(273, 290):                                   # back to the first running set: its cell is replayed again
            out[name].append(r.step([(sa, a[i:i + 1])]).float().cpu().clone())
        r.check_errors()
    assert graph.replays >= 40 and eager.replays == 0
    for e, g2 in zip(out["eager"], out["graph"]):
        assert torch.allclose(e, g2, rtol=0, atol=1e-6 if dtype == torch.float32 else 2e-2), (e - g2).abs().max()


# ------------------------------------------------------------------------------------------------------------------- #
# entry points: engine, command line, trace replay
# ------------------------------------------------------------------------------------------------------------------- #
def test_engine_generates_greedily_like_the_oracle(tmp_path_factory):
    from lite_llama_amd.engine import GenerationEngine, SamplingParams
    from oracle import layered as O

    model, cfg, tens, _ = _model(tmp_path_factory, "flat", torch.float32)
    prompts = [T.prompt(cfg, n, seed=n) for n in (3, 19, 1, 11, 7)]
    engine = GenerationEngine(model, max_tokens=96, max_requests=3, block_size=8, max_step_tokens=10, device=DEV)
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=6))
    for p, o in zip(prompts, outs):
        assert o == O.greedy(cfg, tens, p, 6)
    captured = GenerationEngine(model, max_tokens=96, max_requests=3, block_size=8, max_step_tokens=10, device=DEV, capture_decode=True)
    assert captured.generate(prompts, SamplingParams(max_new_tokens=6)) == outs and captured.runner.replays > 0
    assert engine.runner.cache.free_blocks == engine.runner.total_blocks and engine.runner.free_slots == 3
    sampled = engine.generate(prompts[:2], SamplingParams(max_new_tokens=5, temperature=0.8, top_p=0.9, repetition_penalty=1.2))
    assert [len(s) for s in sampled] == [5, 5] and all(0 <= t < cfg["vocab"] for s in sampled for t in s)


def test_command_line_generate_and_trace_replay(tmp_path_factory, tmp_path):
    from oracle import layered as O

    _, cfg, tens, folder = _model(tmp_path_factory, "flat", torch.float32)
    prompt = T.prompt(cfg, 9, seed=4)
    env = dict(os.environ, PYTHONPATH=ROOT)
    done = subprocess.run([sys.executable, "-m", "lite_llama_amd", "generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "4"],
                          capture_output=True, text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads(done.stdout.strip().splitlines()[-1])
    assert line["prompt"] == prompt and line["generated"] == O.greedy(cfg, tens, prompt, 4)

    a, b = T.prompt(cfg, 21, seed=8), T.prompt(cfg, 6, seed=9)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:13], "want": [0, 12]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [3]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[13:20], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[20:], "want": [0]}, {"id": "c", "tokens": b, "want": [5]}], "end": ["a", "c"]}]
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                          text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [l for l in done.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    import numpy as np

    la, lb = O.forward(cfg, tens, a)[0], O.forward(cfg, tens, b)[0]
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")).view(-1, cfg["vocab"])
    _close(read(0), la[[0, 12]], 2e-5)
    _close(read(1), lb[[5]], 2e-5)
    assert not (out / "2.f32").exists()
    _close(read(3), torch.stack([la[20], lb[5]]), 2e-5)
