"""Plain whole-sequence float64 evaluation of a Purozen model: one function per mechanism, numpy only,
no code shared with the package.  ``w`` maps checkpoint tensor names to float64 arrays, ``cfg`` is the
config.json dict; a sequence is evaluated from position 0 in one go (no cache, no state hand-over)."""
import math

import numpy as np


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm(x, weight, eps):
    """RMS norm whose weight is stored around zero."""
    return rms(x, eps) * (1.0 + weight)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_ff(h, w, pre):
    return gelu_tanh(h @ w[pre + "up"].T) @ w[pre + "down"].T


def softmax_rows(s, visible):
    s = np.where(visible, s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(-1, keepdims=True)


def sigmoid_attention(h, w, pre, m):
    """Causal attention without positions and without softmax: the weight of key j <= i is
    sigmoid(q_i . k_j * scale + pb[head]); the weights are not normalised."""
    T = h.shape[0]
    H, G, D, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, D)
    k = (h @ w[pre + "k"].T).reshape(T, G, D)
    v = (h @ w[pre + "v"].T).reshape(T, G, P)
    causal = np.tril(np.ones((T, T), dtype=bool))
    out = np.zeros((T, H, P))
    for hd in range(H):
        g = hd // (H // G)
        s = q[:, hd] @ k[:, g].T * m["scale"] + w[pre + "pb"][hd]
        out[:, hd] = np.where(causal, sigmoid(s), 0.0) @ v[:, g]
    return out.reshape(T, H * P) @ w[pre + "o"].T


def min_gru(h, w, pre):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t from S = 0, gates from the current token only; the candidate is
    u + 1/2 for u >= 0 and sigmoid(u) below; output W_o (S_t * silu(W_g h_t))."""
    z = sigmoid(h @ w[pre + "z"].T + w[pre + "z.b"])
    u = h @ w[pre + "x"].T + w[pre + "x.b"]
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    g = h @ w[pre + "g"].T
    S = np.zeros(z.shape[1])
    states = np.zeros_like(z)
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        states[t] = S
    return (states * g * sigmoid(g)) @ w[pre + "o"].T


def parallel_mixer(h, w, pre, m):
    left = sigmoid_attention(h, w, pre + "left.", m["left"])
    right = min_gru(h, w, pre + "right.")
    return m["left_scale"] * left + m["right_scale"] * right


def rotate_half(x, rot):
    """x [T, heads, dim]; the first rot['dims'] entries of each head are rotated, entry i with entry
    i + dims/2, by the angle position * base^(-2i/dims) / scaling.factor."""
    if not rot:
        return x
    T = x.shape[0]
    n = rot["dims"]
    i = np.arange(n // 2)
    f = rot["base"] ** (-2.0 * i / n)
    sc = rot.get("scaling")
    if sc:
        f = f / sc["factor"]
    a = np.arange(T)[:, None] * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    out = x.copy()
    u, v = x[..., :n // 2], x[..., n // 2:n]
    out[..., :n // 2] = u * c - v * s
    out[..., n // 2:n] = v * c + u * s
    return out


def window_attention(h, w, pre, m, eps, v_first):
    """Softmax attention with rotated, then unit-RMS q and k; position i sees j <= i with
    i - j < mask.size or j < mask.keep_first.  Returns (output, the values of this layer as projected);
    with ``v_first`` given the values are blended with it before use."""
    T = h.shape[0]
    H, G, D, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(rotate_half((h @ w[pre + "q"].T).reshape(T, H, D), m.get("rot")), eps)
    k = rms(rotate_half((h @ w[pre + "k"].T).reshape(T, G, D), m.get("rot")), eps)
    v_own = h @ w[pre + "v"].T                     # [T, G * P]: blended entry by entry, whatever the head split
    v = v_own
    if v_first is not None:
        lam = float(w[pre + "vmix"])
        v = (1.0 - lam) * v_own + lam * v_first
    v = v.reshape(T, G, P)
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    mask = m.get("mask") or {}
    vis = j <= i
    if mask.get("size"):
        vis &= (i - j < mask["size"]) | (j < mask.get("keep_first", 0))
    out = np.zeros((T, H, P))
    for hd in range(H):
        g = hd // (H // G)
        out[:, hd] = softmax_rows(q[:, hd] @ k[:, g].T * m["scale"], vis) @ v[:, g]
    return out.reshape(T, H * P) @ w[pre + "o"].T, v_own


def latent_attention(h, w, pre, m, eps):
    """Keys and values are up-projections of one normed latent per token; causal softmax, no positions."""
    T = h.shape[0]
    H, D, P = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, D)
    c = rms(h @ w[pre + "dkv"].T, eps) * w[pre + "dkv.norm"]
    k = (c @ w[pre + "uk"].T).reshape(T, H, D)
    v = (c @ w[pre + "uv"].T).reshape(T, H, P)
    causal = np.tril(np.ones((T, T), dtype=bool))
    out = np.zeros((T, H, P))
    for hd in range(H):
        out[:, hd] = softmax_rows(q[:, hd] @ k[:, hd].T * m["scale"], causal) @ v[:, hd]
    return out.reshape(T, H * P) @ w[pre + "o"].T


def as_arrays(w):
    """Checkpoint tensors (torch, any dtype) -> float64 arrays."""
    return {k: (v if isinstance(v, np.ndarray) else v.double().cpu().numpy()) for k, v in w.items()}


def greedy(cfg, w, prompt, n):
    """``n`` greedy tokens after ``prompt``, each from a whole-sequence evaluation."""
    w = as_arrays(w)
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, w, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the residual stream after every layer."""
    w = as_arrays(w)
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    v_first = None
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = norm(x, w[p + "norm1"], eps)
        m = spec["mixer"]
        if spec["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", m)
        elif spec["type"] == "attention":
            y, v_own = window_attention(h, w, p + "mix.", m, eps, v_first if m.get("v_mix") else None)
            if m.get("v_mix") and v_first is None:
                v_first = v_own
        elif spec["type"] == "latent_attention":
            y = latent_attention(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(spec["type"])
        x = x + sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"]) * y
        if spec.get("mlp"):
            h = norm(x, w[p + "norm2"], eps)
            x = x + sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"]) * dense_ff(h, w, p + "mlp.")
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm(x, w["final.norm"], eps) @ w["embed"].T
