"""Small random checkpoints of the layered family for tests: configurations, tensors under the checkpoint's names (values
exactly representable in bfloat16, so a bf16 file holds the same numbers the float64 oracle reads), files on disk."""

import json
import os

import torch


def attention(heads, kv_heads, dim, vdim, ff=0, temp=None, scale=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if temp is not None:
        mixer["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def hgrn2(heads, dim, vdim, ff=0):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width, vocab, loop=None, eps=1e-5):
    cfg = {"architecture": "Rakevik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


CONFIGS = {
    # a loop that starts at layer 0 and runs three times; grouped heads; value width != key width; one head
    "loop0": config([attention(4, 2, 16, 8, ff=96, temp=(0.4, 5)), hgrn2(2, 24, 16), attention(2, 1, 8, 24, ff=72),
                     hgrn2(1, 8, 40, ff=80)], width=64, vocab=97, loop=(0, 2, 3)),
    # no loop at all, feed-forward on the recurrent layer only, every attention head its own key/value head
    "flat": config([hgrn2(3, 16, 16, ff=64), attention(3, 3, 16, 16, temp=(0.25, 3))], width=48, vocab=61, eps=1e-6),
    # a loop that runs once (the entry projection still applies), odd widths
    "once": config([hgrn2(2, 12, 20), attention(5, 1, 12, 20, ff=56, temp=(0.3, 7)), hgrn2(2, 20, 12, ff=40),
                    attention(2, 2, 24, 8)], width=40, vocab=53, loop=(1, 3, 1)),
}


def tensors(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def uni(*shape, lo=0.0, hi=1.0):
        return (torch.rand(*shape, generator=g) * (hi - lo) + lo).to(torch.bfloat16).float()

    def lin(out, inp):
        return rnd(out, inp, std=inp ** -0.5)

    t = {"embed": rnd(V, W), "final.norm": rnd(W, std=0.1, mean=1.0), "head": lin(V, W)}
    if cfg.get("loop"):
        t["loop.in"] = lin(W, 2 * W)
        t["loop.step"] = rnd(cfg["loop"]["times"], W, std=0.3)
    for i, entry in enumerate(cfg["layers"]):
        p, m = f"l{i}.", entry["mixer"]
        t[p + "norm1"] = rnd(W, std=0.1, mean=1.0)
        t[p + "shift"] = uni(W, lo=0.0, hi=0.9)
        if entry["type"] == "hgrn2":
            qk, v = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            t[p + "mix.q"], t[p + "mix.f"], t[p + "mix.v"] = lin(qk, W), lin(qk, W), lin(v, W)
            t[p + "mix.f.b"] = rnd(qk, std=1.0)
            t[p + "mix.lower"] = uni(qk, lo=0.0, hi=0.95)
            t[p + "mix.norm"] = rnd(m["vdim"], std=0.1, mean=1.0)
            t[p + "mix.o"] = lin(W, v)
        else:
            q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = lin(q, W), lin(k, W), lin(v, W)
            t[p + "mix.q.norm"] = rnd(m["dim"], std=0.2, mean=1.5)
            t[p + "mix.k.norm"] = rnd(m["dim"], std=0.2, mean=1.5)
            t[p + "mix.sink"] = rnd(m["heads"], std=1.0)
            t[p + "mix.o"] = lin(W, m["heads"] * m["vdim"])
        if entry["mlp"] is not None:
            ff = entry["mlp"]["ff"]
            t[p + "norm2"] = rnd(W, std=0.1, mean=1.0)
            t[p + "mlp.up"], t[p + "mlp.down"] = lin(ff, W), lin(W, ff)
            t[p + "mlp.act"] = rnd(2, std=0.7)
    return t


def write(folder, cfg, tens):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tens.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)


def prompt(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
