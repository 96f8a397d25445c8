"""Plain, slow restatement of the Rukedra design on the CPU, in float64 unless told otherwise: one function per mechanism,
written from the equations, consuming the checkpoint's tensor names and ``config.json`` directly.  It shares no code with
lite_llama_amd/ (no kernels, no model classes, no cache): whole sequences only, a token loop where the definition is a
recurrence, full score matrices where it is attention, every expert evaluated for every token.

Notation: T tokens, W width, H heads, d / r the unrotated / rotated query-key widths of a head, dv its value width, R the
latent width, E experts, eps the norm epsilon.
"""

from __future__ import annotations

import math

import torch


# ------------------------------------------------------------------------------------- #
# norms, activations
# ------------------------------------------------------------------------------------- #
def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def group_rms_norm(x, weight, eps, groups):
    """The last axis in ``groups`` equal consecutive parts, each divided by its own root mean square; then the weight."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * weight


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------- #
# rotation
# ------------------------------------------------------------------------------------- #
def yarn_frequencies(rot):
    """``(f [dims / 2], amplitude)`` of a rotation description ``{"base", "dims", "scaling": {factor, original, fast, slow}}``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(factor) + 1.0


def rotate_pairs(v, positions, rot, angle_dtype=torch.float64):
    """``v [T, ..., n]``: the first ``rot.dims`` entries of the last axis are rotated pair by pair -- entry 2i with entry
    2i + 1 -- by the angle ``position * f_i``; cos and sin carry the amplitude.  The rest passes unchanged.  ``angle_dtype``:
    the precision in which frequency and angle are held (the design computes them in 32 bits: far out, that rounding of the
    angle is larger than anything else in the rotation)."""
    f, amp = yarn_frequencies(rot)
    dims = int(rot["dims"])
    ang = (positions.to(angle_dtype)[:, None] * f.to(angle_dtype)[None, :]).to(torch.float64)
    cos, sin = (torch.cos(ang) * amp).to(v.dtype), (torch.sin(ang) * amp).to(v.dtype)
    while cos.dim() < v.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


# ------------------------------------------------------------------------------------- #
# mixers
# ------------------------------------------------------------------------------------- #
def latent_attention(h, w, p, m, eps, positions=None):
    """Attention over a shared latent.  ``w[p + name]`` are the mixer's tensors; ``m`` its sizes and constants.  With ``dq``
    the queries pass a normed latent of their own; with ``mask.size`` position i sees the last ``size`` positions only; with
    ``g`` the concatenated heads are gated by sigmoid(W_g h)."""
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T) if positions is None else positions
    if p + "dq" in w:
        q = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T
    else:
        q = h @ w[p + "q"].T
    q = q.view(T, H, d + r)
    dkv = h @ w[p + "dkv"].T
    c = rms_norm(dkv[:, :R], w[p + "dkv.norm"], eps)
    k_rot = rotate_pairs(dkv[:, R:], pos, m["rot"])                         # [T, r], one for all heads
    q_rot = rotate_pairs(q[..., d:], pos, m["rot"])                         # [T, H, r]
    k = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    s = (torch.einsum("thd,shd->hts", q[..., :d], k) + torch.einsum("thr,sr->hts", q_rot, k_rot)) * m["scale"]
    i, j = pos[:, None], pos[None, :]
    seen = j <= i
    if m.get("mask"):
        seen = seen & (i - j < int(m["mask"]["size"]))
    s = s.masked_fill(~seen, float("-inf"))
    o = torch.einsum("hts,shv->thv", torch.softmax(s, -1), v).reshape(T, H * dv)
    if p + "g" in w:
        o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def mingru(h, w, p, state=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t per channel, gates from the current token only; the read-out is gated by silu."""
    z = torch.sigmoid(h @ w[p + "z"].T + w[p + "z.b"])
    u = h @ w[p + "x"].T + w[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(z.shape[1], dtype=h.dtype) if state is None else state
    rows = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        rows.append(S)
    return (torch.stack(rows) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


# ------------------------------------------------------------------------------------- #
# feed-forward
# ------------------------------------------------------------------------------------- #
def gated_mlp(h, w, p, act):
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, router_w, r):
    """``(chosen experts [T, top], their weights [T, top])``: sigmoid scores; experts in ``groups.count`` equal groups of
    neighbours, a group scored by the sum of its two best, only the best ``groups.keep`` groups stay eligible."""
    s = torch.sigmoid(h @ router_w.T)
    T, E = s.shape
    top = int(r["top"])
    eligible = torch.ones_like(s, dtype=torch.bool)
    groups = r.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = s.view(T, count, E // count)
        gscore = per.topk(min(2, E // count), -1).values.sum(-1)
        best = gscore.topk(keep, -1).indices
        gmask = torch.zeros(T, count, dtype=torch.bool)
        gmask.scatter_(1, best, True)
        eligible = gmask[:, :, None].expand(T, count, E // count).reshape(T, E)
    idx = s.masked_fill(~eligible, float("-inf")).topk(top, -1).indices
    chosen = s.gather(1, idx)
    return idx, chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * float(r["scale"])


def moe(h, w, p, mlp):
    idx, weight = route(h, w[p + "router"], mlp["router"])
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=h.dtype)
    for e in range(int(mlp["router"]["experts"])):
        share = (weight * (idx == e)).sum(-1, keepdim=True)                 # 0 where the token did not choose e
        out = out + share * gated_mlp(h, w, f"{p}e{e}.", silu)
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[p + "shared.sg"].T) * gated_mlp(h, w, p + "shared.", silu)
    return out


# ------------------------------------------------------------------------------------- #
# the model
# ------------------------------------------------------------------------------------- #
def forward(config, tensors, tokens, dtype=torch.float64):
    """``(logits [T, vocab], residual stream after every layer [layers, T, W])`` of one whole sequence."""
    w = {k: v.to(dtype) for k, v in tensors.items()}
    eps, groups = float(config["norm"]["eps"]), int(config["norm"].get("groups", 1))

    def norm(x, name):
        return group_rms_norm(x, w[name], eps, groups)

    x = w["embed"][torch.tensor(tokens)]
    after = []
    for i, entry in enumerate(config["layers"]):
        p = f"l{entry.get('weights_of', i)}."
        h = norm(x, p + "norm1")
        if entry["type"] == "mingru":
            y = mingru(h, w, p + "mix.")
        elif entry["type"] in ("latent_attention", "latent_attention_2"):
            y = latent_attention(h, w, p + "mix.", entry["mixer"], eps)
        else:
            raise ValueError(entry["type"])
        y = y * torch.sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"])
        x = x + norm(y, p + "norm1b")
        mlp = entry.get("mlp")
        if mlp is not None:
            h = norm(x, p + "norm2")
            y = moe(h, w, p + "mlp.", mlp) if mlp["kind"] == "moe" else gated_mlp(h, w, p + "mlp.", gelu_tanh)
            y = y * torch.sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"])
            x = x + norm(y, p + "norm2b")
        after.append(x.clone())
    logits = norm(x, "final.norm") @ w["head"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits, torch.stack(after)


def greedy(config, tensors, prompt, new_tokens, dtype=torch.float64):
    """Greedy continuation by re-running the whole sequence for every token."""
    seq = list(prompt)
    for _ in range(new_tokens):
        logits, _ = forward(config, tensors, seq, dtype)
        seq.append(int(torch.argmax(logits[-1])))
    return seq[len(prompt):]
