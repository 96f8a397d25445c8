"""Plain, slow restatement of the layered model family (Rakevik) on the CPU, in float64 unless told otherwise: one function
per mechanism, written from the equations, consuming the CHECKPOINT's tensor names and ``config.json`` directly.  It shares
no code with lite_llama_amd/ (no kernels, no model classes, no cache): whole sequences only, token loops where the
definition is a recurrence, full score matrices where it is attention.

Notation: T tokens, W width, H heads, G key/value heads, dk / dv per-head key / value widths, eps the norm epsilon.
"""

from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def token_shift(h, mu):
    """h_t + (h_(t-1) - h_t) * mu with h_(-1) = 0, over ``[T, W]``."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mu


def softplus(v):
    return math.log1p(math.exp(v))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z / 2."""
    ap, an = softplus(float(p)), 0.5 + softplus(float(q))
    neg = torch.clamp(z, max=0.0)
    return torch.where(z > 0, ap * z * z + z / 2, an * (torch.exp(neg) - 1 - neg) + z / 2)


def hgrn2(h, wq, wf, f_bias, lower, wv, norm_w, wo, heads, dk, dv, eps):
    """Gated linear recurrence, token by token: S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    T = h.shape[0]
    q = torch.nn.functional.silu(h @ wq.T).view(T, heads, dk)
    v = (h @ wv.T).view(T, heads, dv)
    f = (lower + (1 - lower) * torch.sigmoid(h @ wf.T + f_bias)).view(T, heads, dk)
    S = torch.zeros(heads, dk, dv, dtype=h.dtype)
    outs = []
    for t in range(T):
        for a in range(heads):
            S[a] = f[t, a][:, None] * S[a] + (1 - f[t, a])[:, None] * v[t, a][None, :]
        outs.append(torch.stack([S[a].T @ q[t, a] for a in range(heads)]))
    o = rms_norm(torch.stack(outs), norm_w, eps)          # [T, heads, dv], normed over dv
    return o.reshape(T, heads * dv) @ wo.T


def sink_attention(h, wq, wk, wv, q_norm, k_norm, sink, wo, heads, kv_heads, dk, dv, scale, temp_coef, temp_every, eps):
    """Causal softmax attention whose denominator also holds exp(sink_head); queries and keys RMS-normed per head, queries
    scaled by 1 + temp_coef ln(floor((p + 1) / temp_every) + 1)."""
    T = h.shape[0]
    q = rms_norm((h @ wq.T).view(T, heads, dk), q_norm, eps)
    k = rms_norm((h @ wk.T).view(T, kv_heads, dk), k_norm, eps)
    v = (h @ wv.T).view(T, kv_heads, dv)
    out = torch.zeros(T, heads, dv, dtype=h.dtype)
    group = heads // kv_heads
    for t in range(T):
        temp = 1 + temp_coef * math.log(math.floor((t + 1) / temp_every) + 1)
        for a in range(heads):
            g = a // group
            s = (k[: t + 1, g] @ (q[t, a] * temp)) * scale          # [t + 1]
            m = max(float(s.max()), float(sink[a]))
            e = torch.exp(s - m)
            out[t, a] = (e[:, None] * v[: t + 1, g]).sum(0) / (e.sum() + math.exp(float(sink[a]) - m))
    return out.reshape(T, heads * dv) @ wo.T


def run_order(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, 0, False) for i in range(n)]
    a, b = loop["start"], loop["stop"]
    order = [(i, 0, False) for i in range(a)]
    for t in range(loop["times"]):
        order += [(i, t, i == a) for i in range(a, b)]
    return order + [(i, 0, False) for i in range(b, n)]


def forward(config, tensors, tokens, dtype=torch.float64):
    """``(logits [T, vocab], residual stream after every layer run [runs, T, W])`` of one whole sequence."""
    w = {k: v.to(dtype) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    x0 = x.clone()
    after = []
    for index, pass_no, first in run_order(config):
        entry, p = config["layers"][index], f"l{index}."
        m = entry["mixer"]
        if first:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T + w["loop.step"][pass_no]
        h = token_shift(rms_norm(x, w[p + "norm1"], eps), w[p + "shift"])
        if entry["type"] == "hgrn2":
            x = x + hgrn2(h, w[p + "mix.q"], w[p + "mix.f"], w[p + "mix.f.b"], w[p + "mix.lower"], w[p + "mix.v"],
                          w[p + "mix.norm"], w[p + "mix.o"], m["heads"], m["dim"], m["vdim"], eps)
        else:
            temp = m.get("q_temp") or {"coef": 0.0, "every": 1}
            x = x + sink_attention(h, w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.q.norm"], w[p + "mix.k.norm"],
                                   w[p + "mix.sink"], w[p + "mix.o"], m["heads"], m.get("kv_heads", m["heads"]), m["dim"],
                                   m["vdim"], m["scale"], temp["coef"], temp["every"], eps)
        if entry.get("mlp") is not None:
            z = rms_norm(x, w[p + "norm2"], eps) @ w[p + "mlp.up"].T
            x = x + xielu(z, w[p + "mlp.act"][0], w[p + "mlp.act"][1]) @ w[p + "mlp.down"].T
        after.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T, torch.stack(after)


def greedy(config, tensors, prompt, new_tokens, dtype=torch.float64):
    """Greedy continuation by re-running the whole sequence for every token."""
    seq = list(prompt)
    for _ in range(new_tokens):
        logits, _ = forward(config, tensors, seq, dtype)
        seq.append(int(torch.argmax(logits[-1])))
    return seq[len(prompt):]
