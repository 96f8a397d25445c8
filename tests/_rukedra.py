"""Small random Rukedra checkpoints for tests: configurations, tensors under the checkpoint's names (values exactly
representable in bfloat16, so a bf16 file holds the same numbers the float64 oracle reads).  Files are written with
``tests._layered.write``."""

import torch


def rot(dims, base=100.0, factor=4.0, original=64, fast=4.0, slow=0.5):
    return {"base": base, "dims": dims, "scaling": {"factor": factor, "fast": fast, "original": original, "slow": slow}}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, mlp=None, scale=None, **rot_kw):
    """The variant with a query latent, an output gate and a sliding window."""
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
             "mask": {"size": window}, "rot": rot(rot_dim, **rot_kw), "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def latent2(heads, dim, rot_dim, vdim, kv_rank, mlp=None, scale=None, **rot_kw):
    """The variant with directly projected queries, no gate, causal."""
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot(rot_dim, **rot_kw),
             "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    return {"type": "latent_attention_2", "mixer": mixer, "mlp": mlp}


def mingru(width, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None, scale=1.0, shared=0):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def borrowed(entry, owner):
    return dict(entry, weights_of=owner)


def config(layers, width, vocab, groups=1, eps=1e-5, softcap=None):
    cfg = {"architecture": "Rukedra", "layers": layers, "norm": {"eps": eps, "groups": groups}, "vocab": vocab, "width": width}
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


_A = latent(3, 24, 8, 16, 40, 24, 9, mlp=dense(72))
_B = latent(5, 12, 6, 10, 18, 14, 4, mlp=moe(9, 2, 12, groups=(3, 1), scale=1.7, shared=20), base=37.0, factor=2.5, original=24)
CONFIGS = {
    # every mechanism; sizes that are multiples of 8 (the 16-bit matrix-core forms run); a layer without a feed-forward; a layer
    # that borrows another's weights; experts with and without groups / shared expert; three norm groups
    "mix": config([mingru(40, mlp=moe(6, 3, 24, groups=(3, 2), scale=2.0, shared=40)), _A, latent2(2, 16, 16, 24, 24),
                   borrowed(_A, 1), latent2(4, 8, 8, 8, 16, mlp=moe(4, 2, 16))], width=96, vocab=83, groups=3, softcap=9.0),
    # odd sizes: column ranges of the fused projections start off 16-byte borders, a latent row of 26 entries, an expert width
    # that is no multiple of 8, one head, one norm group, a window of 4, no soft cap, the recurrent layer first and last
    "odd": config([mingru(30, mlp=dense(44)), _B, latent2(1, 20, 4, 12, 22, mlp=dense(36), factor=8.0, original=16, fast=2.0),
                   borrowed(_B, 1), mingru(30)], width=60, vocab=47, eps=1e-6),
    # twenty heads on one latent (two column tiles of the grouped decode form), four norm groups, a window longer than a page
    "wide": config([latent2(20, 8, 8, 8, 24, mlp=dense(40)), latent(2, 8, 24, 16, 32, 16, 21, mlp=dense(40), original=512),
                    mingru(64, mlp=moe(8, 4, 8, groups=(2, 1), scale=2.5, shared=8))], width=64, vocab=71, groups=4, softcap=30.0),
    # a layer that borrows from a LATER layer (the shared module is listed under the borrower), two norm groups, top 1 of 2
    "fwd": config([borrowed(mingru(24, mlp=moe(2, 1, 16, shared=8)), 2), latent2(3, 8, 8, 16, 24, mlp=dense(40)),
                   mingru(24, mlp=moe(2, 1, 16, shared=8)), latent(2, 16, 8, 8, 16, 8, 3)], width=48, vocab=59, groups=2),
}


def tensors(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, std=gain * inp ** -0.5)

    def norm(n):
        return rnd(n, std=0.1, mean=1.0)

    def glu(t, p, ff):
        t[p + "gate"], t[p + "up"], t[p + "down"] = lin(ff, W, 1.5), lin(ff, W, 1.5), lin(W, ff, 1.5)

    t = {"embed": rnd(V, W), "final.norm": norm(W), "head": lin(V, W, 2.0)}
    for i, entry in enumerate(cfg["layers"]):
        if entry.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", entry["mixer"]
        for name in ("norm1", "norm1b"):
            t[p + name] = norm(W)
        t[p + "rg1"], t[p + "rg1.b"] = lin(W, W), rnd(W, std=0.5)
        if entry["type"] == "mingru":
            w = m["width"]
            t[p + "mix.z"], t[p + "mix.x"], t[p + "mix.g"], t[p + "mix.o"] = lin(w, W, 2.0), lin(w, W, 2.0), lin(w, W), lin(W, w)
            t[p + "mix.z.b"], t[p + "mix.x.b"] = rnd(w, std=1.0), rnd(w, std=0.5)
        else:
            H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            if entry["type"] == "latent_attention":
                t[p + "mix.dq"], t[p + "mix.dq.norm"], t[p + "mix.uq"] = lin(m["q_rank"], W), norm(m["q_rank"]), lin(H * (d + r), m["q_rank"], 2.0)
                t[p + "mix.g"] = lin(H * dv, W)
            else:
                t[p + "mix.q"] = lin(H * (d + r), W, 2.0)
            t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = lin(R + r, W, 2.0), norm(R)
            t[p + "mix.uk"], t[p + "mix.uv"], t[p + "mix.o"] = lin(H * d, R, 2.0), lin(H * dv, R), lin(W, H * dv)
        mlp = entry["mlp"]
        if mlp is None:
            continue
        for name in ("norm2", "norm2b"):
            t[p + name] = norm(W)
        t[p + "rg2"], t[p + "rg2.b"] = lin(W, W), rnd(W, std=0.5)
        if mlp["kind"] == "dense":
            glu(t, p + "mlp.", mlp["ff"])
        else:
            t[p + "mlp.router"] = lin(mlp["router"]["experts"], W, 3.0)
            for e in range(mlp["router"]["experts"]):
                glu(t, f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared"):
                glu(t, p + "mlp.shared.", mlp["shared"]["ff"])
                t[p + "mlp.shared.sg"] = lin(1, W, 2.0)
    return t
