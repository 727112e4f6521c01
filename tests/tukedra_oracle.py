"""Plain float64 implementation of the Tukedra design: whole sequences, one function per mechanism,
Python loops where the definition has a recurrence.  It shares no code with the package; the tests
compare the engine (kernels, cache, state slots, scheduler) against it.

``cfg`` is a config.json-shaped dict, ``sd`` a dict of tensors by checkpoint name.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def _w(sd, name):
    return sd[name].to(F64)


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# -- rotary positions ----------------------------------------------------------------------------
def rot_table(rot: Dict):
    """Frequencies [dims / 2] and the factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn(t):
        return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))

    lo = max(math.floor(turn(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, pos: torch.Tensor, rot: Optional[Dict], layout: str) -> torch.Tensor:
    """x [n, heads, D]; pairs (2i, 2i+1) for ``layout="pairs"``, (i, i + dims/2) for ``"half"``."""
    if not rot:
        return x
    dims = int(rot["dims"])
    f, m = rot_table(rot)
    ang = pos.to(F64)[:, None, None] * f[None, None, :]
    c, s = torch.cos(ang) * m, torch.sin(ang) * m
    out = x.clone()
    if layout == "pairs":
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = a * c - b * s
        out[..., dims // 2:dims] = b * c + a * s
    return out


# -- mixers --------------------------------------------------------------------------------------
def decay_scan(q, k, v, decay):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k [n, H, D], v [n, H, P]."""
    n, H, D = q.shape
    S = torch.zeros((H, D, v.shape[2]), dtype=F64)
    g = torch.tensor(decay, dtype=F64)[:, None, None]
    out = []
    for t in range(n):
        S = g * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdp,hd->hp", S, q[t]))
    return torch.stack(out)


def lightning(h, sd, p, m, eps):
    n = h.shape[0]
    H, D, P = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ _w(sd, p + "q").T).view(n, H, D)
    k = silu(h @ _w(sd, p + "k").T).view(n, H, D)
    v = silu(h @ _w(sd, p + "v").T).view(n, H, P)
    o = decay_scan(q, k, v, m["decay"]).reshape(n, H * P)
    o = rms(o, eps) * _w(sd, p + "norm") * torch.sigmoid(h @ _w(sd, p + "g").T)
    return o @ _w(sd, p + "o").T


def retention(h, sd, p, m, eps, pos):
    n = h.shape[0]
    H, D, P = m["heads"], m["dim"], m["vdim"]
    q = rotate((h @ _w(sd, p + "q").T).view(n, H, D), pos, m.get("rot"), "half")
    k = rotate((h @ _w(sd, p + "k").T).view(n, H, D), pos, m.get("rot"), "half") * D ** -0.5
    v = (h @ _w(sd, p + "v").T).view(n, H, P)
    o = rms(decay_scan(q, k, v, m["decay"]), eps).reshape(n, H * P)
    return (o * silu(h @ _w(sd, p + "g").T)) @ _w(sd, p + "o").T


def attention(h, sd, p, m, eps, pos):
    n = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ _w(sd, p + "q").T + _w(sd, p + "q.b")).view(n, H, D)
    k = (h @ _w(sd, p + "k").T + _w(sd, p + "k.b")).view(n, G, D)
    v = k.clone()
    q = rms(rotate(q, pos, m.get("rot"), "pairs"), eps)
    k = rms(rotate(k, pos, m.get("rot"), "pairs"), eps)
    rep = H // G
    kk, vv = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)        # query head h reads head h // rep
    sc = torch.einsum("ihd,jhd->hij", q, kk) * float(m["scale"])
    size = (m.get("mask") or {}).get("size")
    pi, pj = pos[:, None], pos[None, :]
    seen = pj <= pi
    if size is not None:
        seen = seen & (pj // size == pi // size)
    w = torch.softmax(sc.masked_fill(~seen[None], float("-inf")), -1)
    out = torch.einsum("hij,jhd->ihd", w, vv)
    return out.reshape(n, H * D) @ _w(sd, p + "o").T


# -- feed-forwards -------------------------------------------------------------------------------
def dense_ff(h, sd, p):
    return (silu(h @ _w(sd, p + "gate").T) * (h @ _w(sd, p + "up").T)) @ _w(sd, p + "down").T


def expert(h, sd, p):
    return torch.relu(h @ _w(sd, p + "up").T).square() @ _w(sd, p + "down").T


def moe_ff(h, sd, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ _w(sd, p + "router").T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(torch.stack([z[t, e] for e in order]), 0)
        for a, e in enumerate(order):
            out[t] += w[a] * expert(h[t:t + 1], sd, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + expert(h, sd, p + "shared.")
    return out


# -- the model -----------------------------------------------------------------------------------
def sublayer_update(xs: List[torch.Tensor], sd, hc: Optional[str], fn, norm_w, eps):
    """One sublayer on the streams ``xs`` (a single stream without hyper-connections)."""
    if hc is None:
        return [xs[0] + fn(rms(xs[0], eps) * norm_w)]
    win, wout, wmix = _w(sd, hc + "in"), _w(sd, hc + "out"), _w(sd, hc + "mix")
    u = sum(win[s] * xs[s] for s in range(len(xs)))
    y = fn(rms(u, eps) * norm_w)
    return [sum(wmix[s, t] * xs[s] for s in range(len(xs))) + wout[t] * y for t in range(len(xs))]


def forward(cfg: Dict, sd: Dict[str, torch.Tensor], tokens, capture: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] (float64) of one sequence from position 0."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(tokens))
    x0 = _w(sd, "embed")[ids] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    streams = cfg.get("streams")
    xs = [x0.clone() for _ in range(streams)] if streams else [x0]
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        if L["type"] == "lightning":
            fn = lambda h: lightning(h, sd, p + "mix.", m, eps)            # noqa: E731
        elif L["type"] == "retention":
            fn = lambda h: retention(h, sd, p + "mix.", m, eps, pos)       # noqa: E731
        elif L["type"] == "attention":
            fn = lambda h: attention(h, sd, p + "mix.", m, eps, pos)       # noqa: E731
        else:
            raise ValueError(L["type"])
        xs = sublayer_update(xs, sd, p + "hc1." if streams else None, fn, _w(sd, p + "norm1"), eps)
        mlp = L.get("mlp")
        if mlp is not None:
            ff = (lambda h: dense_ff(h, sd, p + "mlp.")) if mlp["kind"] == "dense" else \
                 (lambda h: moe_ff(h, sd, p + "mlp.", mlp))                # noqa: E731
            xs = sublayer_update(xs, sd, p + "hc2." if streams else None, ff, _w(sd, p + "norm2"), eps)
        if capture is not None:
            capture.append(sum(xs))
    x = rms(sum(xs), eps) * _w(sd, "final.norm")
    logits = x @ _w(sd, "head").T * float(cfg.get("logit_scale", 1.0))
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits


def greedy(cfg: Dict, sd: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """``n`` greedy tokens after ``prompt``, each from a whole-sequence forward pass."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, sd, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
