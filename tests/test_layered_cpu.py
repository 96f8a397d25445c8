"""Host side of the layered family without a GPU: configuration reader, run order, checkpoint key translation and coverage,
the scheduler's admission / batching / release decisions (over a runner that records what it is asked)."""

import pytest
import torch

from tests import _layered as T


def test_geometry_and_run_order():
    from lite_llama_amd.model_layers import LayeredGeometry
    from oracle import layered as O

    for name, cfg in T.CONFIGS.items():
        geo = LayeredGeometry.from_config(cfg)
        assert geo.run_order() == O.run_order(cfg), name
        assert geo.width == cfg["width"] and geo.vocab_size == cfg["vocab"] and geo.eps == cfg["norm"]["eps"]
    geo = LayeredGeometry.from_config(T.CONFIGS["loop0"])
    assert [r[0] for r in geo.run_order()] == [0, 1, 0, 1, 0, 1, 2, 3]
    assert [r[2] for r in geo.run_order()] == [True, False, True, False, True, False, False, False]
    assert geo.layers[0].mixer.temp_every == 5 and geo.layers[2].mixer.temp_coef == 0.0
    assert not LayeredGeometry.from_config(T.CONFIGS["flat"]).looped
    with pytest.raises(ValueError):
        LayeredGeometry.from_config(T.config([{"type": "conv", "mixer": {}, "mlp": None}], 8, 8))
    with pytest.raises(ValueError):
        LayeredGeometry.from_config(T.config([T.attention(3, 2, 8, 8)], 8, 8))


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_checkpoint_lands_in_the_fused_parameters(tmp_path, name):
    """Every tensor of the checkpoint is copied exactly once; the members of q|f|v and q|k|v sit in their row ranges."""
    from lite_llama_amd.weights import load_pretrained, model_family

    cfg = T.CONFIGS[name]
    tens = T.tensors(cfg, seed=3)
    folder = T.write(tmp_path / name, cfg, tens)
    assert model_family(cfg) == "rakevik"
    model = load_pretrained(folder, device="cpu", dtype=torch.float32)
    assert sum(p.numel() for p in model.parameters()) == sum(v.numel() for v in tens.values())
    for i, entry in enumerate(cfg["layers"]):
        mixer = model.layers[i].mixer
        m = entry["mixer"]
        if entry["type"] == "hgrn2":
            qk = m["heads"] * m["dim"]
            w = mixer.qfv_proj.weight
            assert torch.equal(w[:qk], tens[f"l{i}.mix.q"]) and torch.equal(w[qk:2 * qk], tens[f"l{i}.mix.f"])
            assert torch.equal(w[2 * qk:], tens[f"l{i}.mix.v"]) and torch.equal(mixer.lower, tens[f"l{i}.mix.lower"])
        else:
            q, k = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            w = mixer.qkv_proj.weight
            assert torch.equal(w[:q], tens[f"l{i}.mix.q"]) and torch.equal(w[q:q + k], tens[f"l{i}.mix.k"])
            assert torch.equal(w[q + k:], tens[f"l{i}.mix.v"]) and torch.equal(mixer.sink, tens[f"l{i}.mix.sink"])
    runs = model.cache_runs()
    assert len(runs) == len(model.run_order) and all(r["shift_width"] == cfg["width"] for r in runs)


def test_missing_and_unknown_tensors_are_reported(tmp_path):
    from lite_llama_amd.weights import load_pretrained

    cfg = T.CONFIGS["flat"]
    tens = T.tensors(cfg)
    short = dict(tens)
    del short["l1.mix.sink"]
    with pytest.raises(ValueError, match="never written"):
        load_pretrained(T.write(tmp_path / "a", cfg, short), device="cpu")
    extra = dict(tens)
    extra["l1.mix.window"] = torch.zeros(3)
    with pytest.raises(ValueError, match="unknown parameter"):
        load_pretrained(T.write(tmp_path / "b", cfg, extra), device="cpu")


class _FakeRunner:
    """Stands in for RaggedRunner: same bookkeeping interface, records the steps, answers logits that make token
    ``(last fed token + 1) % vocab`` the argmax."""

    def __init__(self, max_tokens, max_requests, block):
        self.block_size, self.max_requests = block, max_requests
        self.total_blocks = -(-max_tokens // block)
        self.max_seq_len = self.total_blocks * block
        self.free, self.lens, self.steps, self.released = list(range(max_requests)), {}, [], []

    free_slots = property(lambda self: len(self.free))

    def blocks_for(self, n):
        return -(-n // self.block_size)

    def admit(self):
        s = self.free.pop(0)
        self.lens[s] = 0
        return s

    def release(self, slots):
        for s in slots:
            self.released.append((s, self.lens.pop(s)))
            self.free.append(s)

    def step(self, entries, rows):
        self.steps.append([(s, list(t)) for s, t in entries])
        flat = [t for _, toks in entries for t in toks]
        for s, toks in entries:
            self.lens[s] += len(toks)
        assert sum(self.blocks_for(n) for n in self.lens.values()) <= self.total_blocks
        out = torch.zeros(len(rows), 50)
        for i, r in enumerate(rows):
            out[i, (flat[r] + 1) % 50] = 1.0
        return out

    def check_errors(self):
        pass


def _engine(monkeypatch, max_tokens, max_requests, block, budget):
    from lite_llama_amd import engine as E

    monkeypatch.setattr(E, "RaggedRunner", lambda model, mt, mr, bs, dev, capture_decode=False: _FakeRunner(mt, mr, bs))
    eng = E.GenerationEngine(None, max_tokens, max_requests, block, budget, device="cpu")
    monkeypatch.setattr(eng, "_sample", lambda logits, reqs: [int(v) for v in logits.argmax(-1)])
    return eng, E


def test_scheduler_batches_portions_beside_decode_tokens(monkeypatch):
    eng, E = _engine(monkeypatch, max_tokens=64, max_requests=2, block=8, budget=6)
    p = E.SamplingParams(max_new_tokens=3)
    a = eng.add_request([1, 2, 3, 4], p)
    b = eng.add_request(list(range(10, 19)), p)           # 9 tokens: needs two portions under a budget of 6
    c = eng.add_request([30], p)                          # waits for a slot
    done = eng.run()
    assert done[a] == [5, 6, 7] and done[b] == [19, 20, 21] and done[c] == [31, 32, 33]
    steps = eng.runner.steps
    assert steps[0] == [(0, [1, 2, 3, 4]), (1, [10, 11])]                    # budget 6: the second prompt is cut
    assert steps[1] == [(0, [5]), (1, [12, 13, 14, 15, 16])]                 # decode token first, then the next portion
    assert steps[2] == [(0, [6]), (1, [17, 18])]
    assert all(sum(len(t) for _, t in s) <= 6 for s in steps)
    assert [s for s, _ in eng.runner.released][:1] == [0]                    # a finishes first and frees slot 0 ...
    assert any((0, [30]) in s for s in steps)                                # ... which c takes
    assert sorted(n for _, n in eng.runner.released) == [3, 6, 11]           # prompt + generated - 1 tokens were in the cache
    assert eng.idle and eng.runner.free_slots == 2


def test_scheduler_waits_for_blocks_and_keeps_queue_order(monkeypatch):
    eng, E = _engine(monkeypatch, max_tokens=32, max_requests=4, block=8, budget=64)
    big = eng.add_request(list(range(20)), E.SamplingParams(max_new_tokens=4))     # 3 blocks of 4
    big2 = eng.add_request(list(range(100, 117)), E.SamplingParams(max_new_tokens=2))    # 3 blocks: must wait
    small = eng.add_request([1], E.SamplingParams(max_new_tokens=2))               # would fit, but does not overtake
    eng.step()
    assert len(eng._running) == 1 and len(eng._waiting) == 2
    done = eng.run()
    assert set(done) == {big, big2, small}
    first = next(i for i, s in enumerate(eng.runner.steps) if any(t[:1] == [100] for _, t in s))
    assert first >= 4                                                              # only after big released its blocks
    assert next(i for i, s in enumerate(eng.runner.steps) if any(t == [1] for _, t in s)) >= first
    with pytest.raises(ValueError):
        eng.add_request(list(range(40)), E.SamplingParams(max_new_tokens=1))
