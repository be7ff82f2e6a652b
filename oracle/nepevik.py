"""Plain, slow CPU statement of the Nepevik decoder -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token-by-token loops, no cache, no batching; nothing here is shared with
the engine's model code.  ``logits`` runs a whole token sequence and returns the logits of every
position (and, on request, the residual stream after every layer).

Notation.  x: residual stream [n, width].  A layer is x += N1(mixer(x)); x += N2(ff(x)), where
N(y) = y / sqrt(mean(y^2) + eps) * g with ONE gain g per norm.  Weights are [out, in], applied as W y.
"""
import math
from typing import Dict, List, Optional

import torch

_UNIT_EPS = 1e-6                    # inside the root of a unit-vector normalisation


def scalar_norm(y: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps) * g


def rms(y: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps)


def unit(y: torch.Tensor) -> torch.Tensor:
    return y / torch.sqrt(y.pow(2).sum(-1, keepdim=True) + _UNIT_EPS)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def causal_conv_silu(y: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """y [n, channels]; taps [channels, k], the last column weighs the current token; zeros before
    the start."""
    n, k = y.shape[0], taps.shape[1]
    out = torch.zeros_like(y)
    for t in range(n):
        for j in range(k):
            src = t - (k - 1 - j)
            if src >= 0:
                out[t] += taps[:, j] * y[src]
    return out * torch.sigmoid(out)


def visible(i: int, j: int, window: int, keep_first: int) -> bool:
    return j <= i and (i - j < window or j < keep_first)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], cfg: dict, eps: float,
                    shared_kv=None):
    """-> (output [n, width], (keys, values) as a later layer may reuse them)."""
    n = h.shape[0]
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = rms(h @ w["q"].T, eps) * w["q.norm"]
    if shared_kv is None:
        k = rms(h @ w["k"].T, eps) * w["k.norm"]
        v = h @ w["v"].T
    else:
        k, v = shared_kv
    q, kh, vh = q.view(n, H, d), k.view(n, G, d), v.view(n, G, dv)
    window, keep = cfg["mask"]["size"], cfg["mask"]["keep_first"]
    P = torch.zeros(H, n, n, dtype=h.dtype)
    for g in range(H):
        c = g // (H // G)
        for i in range(n):
            js = [j for j in range(i + 1) if visible(i, j, window, keep)]
            s = torch.stack([(q[i, g] * kh[j, c]).sum() for j in js]) * cfg["scale"]
            P[g, i, js] = torch.softmax(s, 0)
    P = torch.einsum("hg,gij->hij", w["talk"], P)          # heads' weights mixed after the softmax
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for g in range(H):
        out[:, g] = P[g] @ vh[:, g // (H // G)]
    return out.reshape(n, H * dv) @ w["o"].T, (k, v)


def channel_delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], cfg: dict, eps: float) -> torch.Tensor:
    """Delta rule with a gate and one decay per head and key channel."""
    n = h.shape[0]
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = causal_conv_silu(h @ w["q"].T, w["q.conv"]).view(n, G, d)
    k = causal_conv_silu(h @ w["k"].T, w["k.conv"]).view(n, G, d)
    v = causal_conv_silu(h @ w["v"].T, w["v.conv"]).view(n, H, dv)
    q, k = unit(q) * d ** -0.5, unit(k)
    beta = torch.sigmoid(h @ w["b"].T)                                               # [n, H]
    pre = (h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]
    decay = torch.exp(-torch.exp(w["A_log"])[None, :, None] * torch.nn.functional.softplus(pre).view(n, H, d))
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(n, H, dv)
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for t in range(n):
        for a in range(H):
            c = a // (H // G)
            S[a] = decay[t, a][:, None] * S[a]
            u = beta[t, a] * (v[t, a] - S[a].T @ k[t, c])
            S[a] = S[a] + torch.outer(k[t, c], u)
            out[t, a] = S[a].T @ q[t, c]
    out = rms(out, eps) * w["norm"] * gate
    return out.reshape(n, H * dv) @ w["o"].T


def general_delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], cfg: dict, eps: float) -> torch.Tensor:
    """Delta rule with separate decay and removal rate per head and key channel."""
    n = h.shape[0]
    H, d = cfg["heads"], cfg["dim"]
    r, k, v = (h @ w["r"].T).view(n, H, d), (h @ w["k"].T).view(n, H, d), (h @ w["v"].T).view(n, H, d)
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ w["w1"].T) @ w["w2"].T + w["w0"])).view(n, H, d)
    rate = torch.sigmoid(h @ w["a"].T + w["a.b"]).view(n, H, d)
    u = unit(k)
    S = torch.zeros(H, d, d, dtype=h.dtype)
    out = torch.zeros(n, H, d, dtype=h.dtype)
    for t in range(n):
        for a in range(H):
            old = S[a]
            S[a] = decay[t, a][:, None] * old - torch.outer(rate[t, a] * u[t, a], u[t, a] @ old) \
                + torch.outer(k[t, a], v[t, a])
            out[t, a] = S[a].T @ r[t, a]
    out = rms(out, eps).reshape(n, H * d) * w["norm"] * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


def table_moe(h: torch.Tensor, tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    """Experts chosen by a table over token ids, equal weights; a gated shared expert on top."""
    out = torch.zeros_like(h)
    top = cfg["router"]["top"]
    for t, tok in enumerate(tokens):
        for e in w["table"][tok].tolist():
            out[t] += (w[f"e{e}.down"] @ gelu_erf(w[f"e{e}.up"] @ h[t])) / top
    if cfg.get("shared"):
        shared = gelu_erf(h @ w["shared.up"].T) @ w["shared.down"].T
        out = out + torch.sigmoid(h @ w["shared.sg"].T) * shared
    return out


def _sub(sd: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: (v if not v.dtype.is_floating_point else v.to(dtype))
            for k, v in sd.items() if k.startswith(prefix)}


def logits(sd: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], dtype=torch.float64,
           residuals: Optional[list] = None) -> torch.Tensor:
    eps = cfg["norm"]["eps"]
    x = sd["embed"].to(dtype)[torch.tensor(tokens)]
    kv = {}
    for i, layer in enumerate(cfg["layers"]):
        w = _sub(sd, f"l{i}.mix.", dtype)
        m = layer["mixer"]
        if layer["type"] == "attention":
            y, kv[i] = attention_mixer(x, w, m, eps, kv.get(m.get("kv_from")) if "kv_from" in m else None)
        elif layer["type"] == "channel_delta":
            y = channel_delta_mixer(x, w, m, eps)
        elif layer["type"] == "general_delta":
            y = general_delta_mixer(x, w, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + scalar_norm(y, sd[f"l{i}.norm1"].to(dtype), eps)
        if layer.get("mlp") is not None:
            y = table_moe(x, tokens, _sub(sd, f"l{i}.mlp.", dtype), layer["mlp"])
            x = x + scalar_norm(y, sd[f"l{i}.norm2"].to(dtype), eps)
        if residuals is not None:
            residuals.append(x.clone())
    return scalar_norm(x, sd["final.norm"].to(dtype), eps) @ sd["head"].to(dtype).T
