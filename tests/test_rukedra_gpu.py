"""Rukedra on the GPU against the plain CPU restatement (oracle/rukedra.py): each mechanism's kernels alone, then whole
models built from small random checkpoints through the loader, the ragged runner, the paged state cache, the generation
engine and the command line.  float32 runs are held to rounding error; bfloat16 runs to the rounding of their activations.
Where random weights would hide a fault (a key far back, a window's edge), one key is made to dominate."""

import json
import os
import subprocess
import sys

import pytest
import torch

from tests import _layered as L
from tests import _rukedra as T
from tests.test_layered_gpu import _close, _feed, _step

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def _rt(t, dtype):
    """Random values already rounded to ``dtype``: the oracle and the kernel read the same numbers."""
    return t.to(dtype)


# ------------------------------------------------------------------------------------------------------------------- #
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,groups,parts,shared,gated", [(96, 3, 1, False, True), (60, 1, 3, True, True), (2048, 2, 2, True, True),
                                                             (8192, 2, 1, False, False), (8200, 1, 2, False, True)])
def test_gated_group_norm_sums_gates_norms_adds_and_norms_again(dtype, width, groups, parts, shared, gated):
    from lite_llama_amd.kernels.norm_act import GatedUpdate, gated_group_norm
    from oracle import rukedra as O

    torch.manual_seed(width + parts)
    n, eps = 5, 1e-5
    x = torch.randn(n, width, device=DEV) * 3
    y = _rt(torch.randn(n, parts, width, device=DEV), dtype)
    wide = _rt(torch.randn(n, width + 24, device=DEV) * 2, dtype)       # gate logits = a column range of wider rows
    gate, bias = (wide[:, 17:17 + width], _rt(torch.randn(width, device=DEV), dtype)) if gated else (None, None)
    sh = _rt(torch.randn(n, width, device=DEV), dtype) if shared else None
    sc = torch.rand(n, device=DEV) if shared else None
    pw, nw = _rt(1 + 0.1 * torch.randn(width, device=DEV), dtype), _rt(1 + 0.1 * torch.randn(width, device=DEV), dtype)
    d = lambda t: t.cpu().to(F64)   # noqa: E731
    s = d(y).sum(1)
    if shared:
        s = s + d(sc)[:, None] * d(sh)
    if gated:
        s = s * torch.sigmoid(d(gate) + d(bias))
    want_x = d(x) + O.group_rms_norm(s, d(pw), eps, groups)
    want_h = O.group_rms_norm(want_x, d(nw), eps, groups)
    upd = GatedUpdate(y, pw, gate, bias, sh, sc)
    x1 = x.clone()
    h = gated_group_norm(x1, upd, nw, eps, groups)
    _close(x1, want_x, 2e-6 if dtype == torch.float32 else 2e-2)   # (the 16-bit form takes the hardware exponential in the gate)
    _close(h, want_h, TOL[dtype])
    # only the residual; only the norm; the update of some rows
    x2 = x.clone()
    assert gated_group_norm(x2, upd, None, eps, groups) is None
    assert torch.equal(x2, x1)
    _close(gated_group_norm(x.clone(), None, nw, eps, groups), O.group_rms_norm(d(x), d(nw), eps, groups), TOL[dtype])
    pick = torch.tensor([3, 0], device=DEV)
    x3 = x[pick].contiguous()
    gated_group_norm(x3, upd.rows(pick), nw, eps, groups)
    assert torch.allclose(x3, x1[pick], rtol=0, atol=2e-6 * float(x1.abs().max()))   # (aligned rows take the vector form)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_glu_activations_and_softcap(dtype):
    from lite_llama_amd.kernels.norm_act import glu_act, softcap_
    from oracle import rukedra as O

    rows = _rt(torch.randn(9, 2 * 37 + 5, device=DEV) * 3, dtype)
    g, u = rows[:, :37].cpu().to(F64), rows[:, 37:74].cpu().to(F64)
    _close(glu_act(rows, 37, "gelu_tanh"), O.gelu_tanh(g) * u, TOL[dtype])
    _close(glu_act(rows, 37, "silu"), O.silu(g) * u, TOL[dtype])
    other = _rt(torch.randn(9, 37, device=DEV), dtype)
    _close(glu_act(rows[:, 3:], 37, "sigmoid", up=other), torch.sigmoid(rows[:, 3:40].cpu().to(F64)) * other.cpu().to(F64), TOL[dtype])
    z = _rt(torch.linspace(-40, 40, 301, device=DEV), dtype)
    _close(softcap_(z.clone(), 7.5), 7.5 * torch.tanh(z.cpu().to(F64) / 7.5), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rank,rot,dims,q_rank", [(40, 8, 8, 24), (18, 6, 6, 14), (22, 6, 4, 0), (130, 64, 64, 0)])
def test_latent_rows_are_normed_rotated_at_their_positions_and_written_to_their_cache_rows(dtype, rank, rot, dims, q_rank):
    from lite_llama_amd.kernels.attention import latent_kv_prep, rotate_pairs
    from lite_llama_amd.model_layers import RotarySpec
    from oracle import rukedra as O

    torch.manual_seed(rank)
    desc = T.rot(dims, base=500.0, factor=4.0, original=128)
    freq, amp = RotarySpec.from_config(desc).table()
    freq = torch.tensor(freq, dtype=F64).float().to(DEV)
    seqs = [(0, 0, 4, 0), (2, 4100, 1, 0), (1, 63, 3, 0)]            # a start, a token decoded far out, a portion over a page edge
    table = torch.randperm(3 * 4200)[:3 * 4200].view(3, 4200).to(torch.int32)   # cache rows in random order
    step = _step(seqs, table)
    n = step.num_tokens
    kv_off, ld = q_rank + 3, q_rank + 3 + rank + rot + 5
    rows = _rt(torch.randn(n, ld, device=DEV), dtype)
    wk, wq = _rt(1 + 0.1 * torch.randn(rank, device=DEV), dtype), _rt(1 + 0.1 * torch.randn(max(q_rank, 1), device=DEV), dtype)
    cache = torch.zeros(3 * 4200, rank + rot, dtype=dtype, device=DEV)
    cq = latent_kv_prep(rows, kv_off, rank, rot, wk, 1e-5, freq, dims // 2, amp, step, cache, q_off=0, q_rank=q_rank,
                        q_norm_weight=wq[:q_rank] if q_rank else None)
    pos = step.tok_pos.cpu().long()
    r64 = rows.cpu().to(F64)
    got = cache[step.select.long()]
    _close(got[:, :rank], O.rms_norm(r64[:, kv_off:kv_off + rank], wk.cpu().to(F64), 1e-5), TOL[dtype])
    _close(got[:, rank:], O.rotate_pairs(r64[:, kv_off + rank:kv_off + rank + rot], pos, desc, torch.float32), TOL[dtype])
    if q_rank:
        _close(cq, O.rms_norm(r64[:, :q_rank], wq[:q_rank].cpu().to(F64), 1e-5), TOL[dtype])
    assert int((cache.abs().sum(-1) > 0).sum()) == n                  # nothing else was touched
    heads, d = 3, 5
    q = _rt(torch.randn(n, heads * (d + rot) + 2, device=DEV), dtype)[:, :heads * (d + rot)].view(n, heads, d + rot)
    out = torch.zeros(n, heads, rank + rot, dtype=dtype, device=DEV)
    rotate_pairs(q, d, rot, freq, dims // 2, amp, step, out, rank)
    _close(out[:, :, rank:], O.rotate_pairs(q[:, :, d:].cpu().to(F64), pos, desc, torch.float32), TOL[dtype])
    assert float(out[:, :, :rank].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 30, 300])
@pytest.mark.parametrize("long", [False, True])
def test_mingru_carries_state_across_steps_and_ignores_stale_slots(dtype, width, long):
    """Short runs take the plain walk; runs of 128 tokens and more are walked in chunks of 32 side by side (a last chunk of 8
    and of 22 tokens, a neighbour that brings 1 or 3 tokens into the same launch and carries its state through it)."""
    from lite_llama_amd.kernels.recurrent import mingru_scan
    from oracle import rukedra as O

    torch.manual_seed(width)
    lens = {1: 353, 0: 154} if long else {1: 23, 0: 11}
    plans = {False: [[(1, 0, 9), (0, 0, 1)], [(0, 1, 1), (1, 9, 1)], [(1, 10, 13), (0, 2, 9)]],
             True: [[(1, 0, 200), (0, 0, 1)], [(1, 200, 3), (0, 1, 150)], [(0, 151, 3), (1, 203, 150)]]}
    rows = {s: _rt(torch.randn(n, 3 * width + 7, device=DEV) * 2, dtype) for s, n in lens.items()}
    zb, xb = _rt(torch.randn(width, device=DEV), dtype), _rt(torch.randn(width, device=DEV), dtype)
    eye = torch.eye(width, dtype=F64)
    want = {}
    for s, r in rows.items():   # the oracle's projections are identities: its input is the rows themselves
        r64 = r.cpu().to(F64)
        w = {"z": torch.cat([eye, torch.zeros(width, 2 * width + 7, dtype=F64)], 1), "z.b": zb.cpu().to(F64),
             "x": torch.cat([torch.zeros(width, width, dtype=F64), eye, torch.zeros(width, width + 7, dtype=F64)], 1), "x.b": xb.cpu().to(F64),
             "g": torch.cat([torch.zeros(width, 2 * width, dtype=F64), eye, torch.zeros(width, 7, dtype=F64)], 1), "o": eye}
        want[s] = O.mingru(r64, w, "")
    state = torch.full((3, width), 7.0, device=DEV)                     # stale: a sequence that starts must not read it
    plan = plans[long]
    got = {s: [] for s in lens}
    for seqs in plan:
        step = _step([(s, f, c, 0) for s, f, c in seqs])
        batch = torch.cat([rows[s][f:f + c] for s, f, c in seqs])
        out = mingru_scan(batch, width, zb, xb, step, state)
        at = 0
        for s, f, c in seqs:
            got[s].append(out[at:at + c])
            at += c
    for s in lens:
        _close(torch.cat(got[s]), want[s], TOL[dtype])
    assert torch.all(state[2] == 7.0)


def _window_case(dtype, heads, rank, rot, total, plan, window, hot=None, scale=0.3):
    """Queries against a latent cache (values = the first ``rank`` columns of the key rows) through the attention kernels,
    fed by ``plan`` (steps of ``(slot, first, count)``); returns (got, want) of the slot-1 sequence."""
    from lite_llama_amd.kernels.attention import ragged_attention

    torch.manual_seed(total + heads)
    dk = rank + rot
    q = torch.randn(total, heads, dk)
    k = torch.randn(total, dk)
    if hot is not None:        # one key whose score towers over the rest for every query that may see it
        u = torch.nn.functional.normalize(torch.randn(dk), dim=0)
        k[hot] = 9.0 * u
        q = q + 9.0 * u
    q, k = q.to(dtype), k.to(dtype)
    rows_total = 2 * total + 64
    table = torch.randperm(rows_total)[:2 * total].view(2, total).to(torch.int32).to(DEV)
    cache = torch.randn(rows_total, 1, dk).to(dtype).to(DEV)
    cache[table[1].long(), 0] = k.to(DEV)
    cache[table[0].long(), 0] = torch.randn(total, dk).to(dtype).to(DEV)   # a neighbour in slot 0
    q0 = torch.randn(total, heads, dk).to(dtype)
    got = []
    for seqs in plan:
        step = _step([(s, f, c, 0) for s, f, c in seqs], table.cpu())
        qs = torch.cat([(q if s == 1 else q0)[f:f + c] for s, f, c in seqs]).to(DEV).contiguous()
        out = ragged_attention(qs, cache, cache[:, :, :rank], scale, step, table, window=window)
        at = 0
        for s, f, c in seqs:
            if s == 1:
                got.append(out[at:at + c])
            at += c
    q64, k64 = q.to(F64), k.to(F64)
    s = torch.einsum("thd,sd->hts", q64, k64) * scale
    i, j = torch.arange(total)[:, None], torch.arange(total)[None, :]
    seen = (j <= i) & ((i - j < window) if window else True)
    want = torch.einsum("hts,sv->thv", torch.softmax(s.masked_fill(~seen, float("-inf")), -1), k64[:, :rank]).reshape(total, heads * rank)
    return torch.cat(got), want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 50])
def test_latent_rows_wider_than_the_matrix_core_forms_serve(dtype, window):
    """A latent of 272 + 16 entries per row (more than the 16-bit matrix-core forms take): the plain form with eight value
    columns per lane, prompt portion and decoded tokens."""
    total = 90
    plan = [[(1, 0, 70), (0, 0, 2)]] + [[(1, 70 + i, 1), (0, 2 + i, 1)] for i in range(20)]
    got, want = _window_case(dtype, 2, 272, 16, total, plan, window, hot=33, scale=0.15)
    _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rank,rot", [(40, 8), (22, 4)])             # (26 entries per row: the 16-bit matrix-core form does not apply)
@pytest.mark.parametrize("hot", [0, 3, 63, 64, 255, 256, 600])
def test_one_far_key_reaches_prompt_portions_and_decoded_tokens(dtype, rank, rot, hot):
    """Causal attention over 700 positions in pages of 64; the key at ``hot`` decides every later token's output."""
    total = 700
    plan = [[(1, 0, 300), (0, 0, 5)], [(1, 300, 390)]] + [[(0, 5 + i, 1), (1, 690 + i, 1)] for i in range(10)]
    got, want = _window_case(dtype, 3, rank, rot, total, plan, 0, hot=hot)
    _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)
    assert (got[hot + 1:].float().cpu() - want[hot + 1:]).abs().max() < 0.1 * want.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rank,rot", [(40, 8), (22, 4)])
@pytest.mark.parametrize("window,hot", [(1, 5), (9, 40), (21, 300), (64, 191), (100, 256), (300, 70)])
def test_window_edge_in_prompts_and_in_decoding(dtype, rank, rot, window, hot):
    """The dominating key sits at ``hot``: position hot + window - 1 still sees it, hot + window does not.  The edge is crossed
    once inside a prompt portion and (in a second run) by decoded tokens; windows shorter and longer than a tile, a page and
    a context partition."""
    total = hot + window + 40
    edge = hot + window
    prompt = [[(1, 0, 7), (0, 0, 3)], [(1, 7, total - 7)]]
    decode = [[(1, 0, edge - 3)]] + [[(1, i, 1), (0, i - edge + 3, 1)] for i in range(edge - 3, total)]
    for plan in (prompt, decode):
        got, want = _window_case(dtype, 4, rank, rot, total, plan, window, hot=hot)
        _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)
        gap = (want[edge - 1] - want[edge]).abs().max()              # the outputs on the two sides of the edge differ grossly
        assert gap > 1.0 and (got[edge - 1:edge + 1].float().cpu() - want[edge - 1:edge + 1]).abs().max() < 0.05 * gap


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,groups,width", [(6, 3, (3, 2), 96), (9, 2, (3, 1), 60), (4, 2, None, 33), (64, 6, (8, 3), 128),
                                                      (1, 1, None, 16), (8, 8, (2, 2), 40), (5, 2, (5, 3), 24)])   # (the last: groups of one)
def test_group_router_chooses_like_the_oracle(dtype, experts, top, groups, width):
    from lite_llama_amd.kernels.fused_moe import group_router
    from oracle import rukedra as O

    torch.manual_seed(experts * top)
    n = 41
    h = _rt(torch.randn(n, width + 8, device=DEV), dtype)[:, :width]   # (row-strided input)
    wr = _rt(torch.randn(experts, width, device=DEV) * 3 * width ** -0.5, dtype)
    we = _rt(torch.randn(1, width, device=DEV) * width ** -0.5, dtype)
    router = {"experts": experts, "top": top, "scale": 1.9}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    ids, weights, extra = group_router(h, wr, top, *(groups or (1, 1)), route_scale=1.9, extra_weight=we)
    want_ids, want_w = O.route(h.cpu().to(F64), wr.cpu().to(F64), router)
    assert torch.equal(ids.cpu().long(), want_ids)                      # slot k = the k-th best
    _close(weights, want_w, 1e-5)
    _close(extra, torch.sigmoid(h.cpu().to(F64) @ we.cpu().to(F64).T)[:, 0], 1e-5)
    assert group_router(h, wr, top, *(groups or (1, 1)))[2] is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,width,experts,top,ff", [(37, 64, 6, 3, 24), (5, 60, 9, 2, 12), (1, 96, 4, 4, 40), (300, 32, 3, 1, 8),
                                                    (600, 64, 3, 2, 24), (1100, 136, 4, 2, 72)])   # (the last two: blocks of 128 rows)
def test_expert_products_per_slot(dtype, n, width, experts, top, ff):
    from lite_llama_amd.kernels.fused_moe import sparse_glu_experts
    from oracle import rukedra as O

    torch.manual_seed(n + ff)
    h = _rt(torch.randn(n, width, device=DEV), dtype)
    wgu = _rt(torch.randn(experts, 2 * ff, width, device=DEV) * width ** -0.5, dtype)
    wd = _rt(torch.randn(experts, width, ff, device=DEV) * ff ** -0.5, dtype)
    ids = torch.stack([torch.randperm(experts)[:top] for _ in range(n)]).to(torch.int32).to(DEV)
    if n == 300:
        ids[:] = 2                                                       # everybody on one expert: the others' runs are empty
    weights = torch.rand(n, top, device=DEV) + 0.1
    got = sparse_glu_experts(h, wgu, wd, ids, weights)
    h64 = h.cpu().to(F64)
    want = torch.zeros(n, top, width, dtype=F64)
    for e in range(experts):
        w = {"gate": wgu[e, :ff].cpu().to(F64), "up": wgu[e, ff:].cpu().to(F64), "down": wd[e].cpu().to(F64)}
        full = O.gated_mlp(h64, w, "", O.silu)
        hit = (ids.cpu() == e)
        want[hit] = (full[:, None, :] * weights.cpu().to(F64)[:, :, None])[hit]
    _close(got, want, TOL[dtype])


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
        folder = L.write(tmp_path_factory.mktemp(name), cfg, tens)
        _MODELS[key] = (load_pretrained(folder, device=DEV, dtype=dtype), cfg, tens, folder)
    return _MODELS[key]


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_whole_prompt_layers_and_logits(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import rukedra as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 45)
    want, layers = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 64, 2, block_size=16, device=DEV)
    got_layers = []
    got = runner.step([(runner.admit(), toks)], list(range(len(toks))), collect_layers=got_layers)
    runner.check_errors()
    assert len(got_layers) == len(cfg["layers"])
    for i, layer in enumerate(got_layers):
        _close(layer, layers[i], 2e-5)
    _close(got, want, 2e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_whole_prompts_take_the_expanded_form_and_agree_with_the_oracle_and_with_portions(tmp_path_factory, name, monkeypatch):
    """Prompts of 64 tokens and more that start their sequences expand keys / values per head from the step's own latent rows
    instead of reading them through the absorbed form: two unequal prompts in one step, and a long first portion followed by
    portions and decoded tokens that read the same rows from the cache."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.model_layers import LatentAttention
    from oracle import rukedra as O

    calls = []
    plain = LatentAttention._expanded
    monkeypatch.setattr(LatentAttention, "_expanded", lambda self, *a: (calls.append(1), plain(self, *a))[1])
    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    a, b = L.prompt(cfg, 150, seed=11), L.prompt(cfg, 67, seed=12)
    wa, wb = O.forward(cfg, tens, a)[0], O.forward(cfg, tens, b)[0]
    runner = RaggedRunner(model, 512, 3, block_size=16, device=DEV)
    sa, sb = runner.admit(), runner.admit()
    got = runner.step([(sa, a), (sb, b)], list(range(217)))
    latent_layers = sum(1 for e in cfg["layers"] if e["type"] != "mingru")
    assert len(calls) == latent_layers
    _close(got[:150], wa, 2e-5)
    _close(got[150:], wb, 2e-5)
    runner.release([sa, sb])
    _close(_feed(runner, runner.admit(), a, [70, 3, 40, 1]), wa, 2e-5)      # the first portion expanded, the rest absorbed
    assert len(calls) == 2 * latent_layers
    runner.check_errors()
    half, _, _, _ = _model(tmp_path_factory, name, torch.bfloat16)
    r16 = RaggedRunner(half, 512, 2, block_size=16, device=DEV)
    whole = _feed(r16, r16.admit(), a, [150]).float().cpu()                   # expanded
    parts = _feed(r16, r16.admit(), a, [50, 50, 50]).float().cpu()            # absorbed
    err = lambda x, y: (x.to(F64) - y.to(F64)).pow(2).mean(-1).sqrt().median().item()   # noqa: E731
    assert err(whole, wa) < 0.06 * wa.std().item() and err(parts, whole) < 0.04 * wa.std().item()


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
@pytest.mark.parametrize("sizes", [[1], [2], [3, 2, 7, 1, 16, 5], [40, 1]])
def test_portions_and_token_by_token_decoding_equal_the_whole_prompt(tmp_path_factory, name, sizes):
    """Portions down to two tokens, pure token-by-token decoding from the first token on, and a long portion followed by
    decoding; pages of 8 tokens, so portions, windows and pages start and end inside one another."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import rukedra as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 58, seed=1)
    want, _ = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 64, 2, block_size=8, device=DEV)
    _close(_feed(runner, runner.admit(), toks, sizes), want, 2e-5)
    runner.check_errors()


def test_unequal_requests_in_one_batch_equal_each_alone_and_freed_pages_and_slots_are_used_again(tmp_path_factory):
    """Four requests of different lengths ride together in changing portions, three slots and a pool that only holds them
    because finished requests give their pages back; a late request takes over a used slot (with its stale recurrent state)
    and used pages."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import rukedra as O

    model, cfg, tens, _ = _model(tmp_path_factory, "mix", torch.float32)
    lens = {"a": 41, "b": 9, "c": 26, "d": 33}
    toks = {k: L.prompt(cfg, n, seed=ord(k)) for k, n in lens.items()}
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
    assert slot["d"] in (slot["a"], slot["b"], slot["c"])
    assert runner.cache.free_blocks == runner.total_blocks
    for name in lens:
        _close(torch.cat(got[name]), want[name], 2e-5)


@pytest.mark.parametrize("name", ["odd", "wide"])
def test_long_decoding_past_windows_and_over_many_pages(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import rukedra as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 150, seed=5)
    want, _ = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 160, 1, block_size=16, device=DEV)
    _close(_feed(runner, runner.admit(), toks, [6, 1]), want, 3e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_bfloat16_model_tracks_the_oracle_and_its_own_portions(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import rukedra as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.bfloat16)
    toks = L.prompt(cfg, 70, seed=2)
    want, _ = O.forward(cfg, tens, toks)
    runner = RaggedRunner(model, 160, 2, block_size=16, device=DEV)
    whole = _feed(runner, runner.admit(), toks, [70]).float().cpu()
    parts = _feed(runner, runner.admit(), toks, [2, 9, 1, 1, 30, 1]).float().cpu()
    spread = want.std().item()
    # medians over the tokens: a token whose router sees two experts within a rounding step of each other may choose the other
    err = lambda a, b: (a.to(F64) - b.to(F64)).pow(2).mean(-1).sqrt().median().item()   # noqa: E731
    assert err(whole, want) < 0.06 * spread
    assert err(parts, whole) < 0.04 * spread


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_replay_like_eager_ones(tmp_path_factory, dtype):
    from lite_llama_amd.executor.ragged import RaggedRunner

    model, cfg, _, _ = _model(tmp_path_factory, "mix", dtype)
    a, b = L.prompt(cfg, 290, seed=21), L.prompt(cfg, 40, seed=22)
    eager = RaggedRunner(model, 512, 2, block_size=16, device=DEV)
    graph = RaggedRunner(model, 512, 2, block_size=16, device=DEV, capture_decode=True)
    out = {"eager": [], "graph": []}
    for name, r in (("eager", eager), ("graph", graph)):
        sa, sb = r.admit(), r.admit()
        r.step([(sa, a[:240])], [])
        for i in range(240, 262):                                   # one sequence decoding across a partition edge
            out[name].append(r.step([(sa, a[i:i + 1])]).float().cpu().clone())
        r.step([(sa, a[262:263]), (sb, b[:30])], [])
        for i in range(10):                                         # two sequences decoding together
            out[name].append(r.step([(sa, a[263 + i:264 + i]), (sb, b[30 + i:31 + i])]).float().cpu().clone())
        r.release([sb])
        for i in range(273, 290):
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
    from oracle import rukedra as O

    model, cfg, tens, _ = _model(tmp_path_factory, "odd", torch.float32)
    prompts = [L.prompt(cfg, n, seed=n) for n in (3, 19, 1, 11, 7)]
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
    from oracle import rukedra as O

    _, cfg, tens, folder = _model(tmp_path_factory, "wide", torch.float32)
    prompt = L.prompt(cfg, 9, seed=4)
    env = dict(os.environ, PYTHONPATH=ROOT)
    done = subprocess.run([sys.executable, "-m", "lite_llama_amd", "generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "4"],
                          capture_output=True, text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads(done.stdout.strip().splitlines()[-1])
    assert line["prompt"] == prompt and line["generated"] == O.greedy(cfg, tens, prompt, 4)

    a, b = L.prompt(cfg, 31, seed=8), L.prompt(cfg, 6, seed=9)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:13], "want": [0, 12]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [3]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[13:30], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[30:], "want": [0]}, {"id": "c", "tokens": b, "want": [5]}], "end": ["a", "c"]}]
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                          text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [ln for ln in done.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    import numpy as np

    la, lb = O.forward(cfg, tens, a)[0], O.forward(cfg, tens, b)[0]
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")).view(-1, cfg["vocab"])   # noqa: E731
    _close(read(0), la[[0, 12]], 2e-5)
    _close(read(1), lb[[5]], 2e-5)
    assert not (out / "2.f32").exists()
    _close(read(3), torch.stack([la[30], lb[5]]), 2e-5)
