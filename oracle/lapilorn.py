"""Plain, slow CPU statement of the Lapilorn decoder -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token-by-token loops, no cache, no batching; nothing here is shared with the
engine's model code.  ``logits`` runs a whole token sequence and returns the logits of every position (and,
on request, the residual stream after every layer).

Notation.  x: residual stream [n, width].  A layer reads ONE norm of the stream for both of its sublayers:
    h = N(x);  x <- x + (mixer(h) + ff(h)),      N(y) = y / sqrt(mean(y^2) + eps) * (1 + w)
Weights are [out, in] and applied as W y.  The logits reuse the embedding table.
"""
import math
from typing import Dict, List, Optional

import torch


def offset_norm(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w)


def plain_norm(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps) * w


def rotary_frequencies(rot: dict) -> List[float]:
    """One frequency per rotated pair, with the wavelength-dependent slowdown of long waves."""
    dims, base = rot["dims"], rot["base"]
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            wavelength = 2.0 * math.pi / f
            if wavelength < sc["original"] / sc["high"]:
                pass
            elif wavelength > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            else:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return out


def rotate(y: torch.Tensor, position: int, freqs: List[float]) -> torch.Tensor:
    """y [heads, size]: neighbours (2i, 2i + 1) of the first 2 * len(freqs) coordinates turn by position * f_i
    (the angle is the fp32 product of the fp32 position and the fp32 frequency, as the design computes it)."""
    out = y.clone()
    for i, f in enumerate(freqs):
        a = (torch.tensor(float(position), dtype=torch.float32) * torch.tensor(f, dtype=torch.float32)).double()
        c, s = torch.cos(a).to(y.dtype), torch.sin(a).to(y.dtype)
        u, v = y[:, 2 * i], y[:, 2 * i + 1]
        out[:, 2 * i] = u * c - v * s
        out[:, 2 * i + 1] = v * c + u * s
    return out


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: Optional[float],
                     window: int = 0, first_position: int = 0) -> torch.Tensor:
    """q [n, H, d] at positions first_position ..; k [m, G, d], v [m, G, dv] from position 0 (already rotated).
    -> [n, H, dv].  Query head a reads key/value head a // (H // G); position i sees j <= i (and i - j < window)."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        pos = first_position + t
        lo = max(0, pos - window + 1) if window else 0
        for a in range(H):
            g = a // (H // G)
            s = (k[lo:pos + 1, g] @ q[t, a]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            out[t, a] = torch.softmax(s, 0) @ v[lo:pos + 1, g]
    return out


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, shared_kv=None):
    """-> (output [n, width], (rotated keys, values) as a later layer may reuse them)."""
    n = h.shape[0]
    H, d = m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", d)
    freqs = rotary_frequencies(m["rot"]) if m.get("rot") else []
    q = (h @ w["q"].T).view(n, H, d)
    q = torch.stack([rotate(q[t], t, freqs) for t in range(n)])
    if shared_kv is None:
        k = (h @ w["k"].T).view(n, G, d)
        k = torch.stack([rotate(k[t], t, freqs) for t in range(n)])
        v = (h @ w["v"].T).view(n, G, dv)
    else:
        k, v = shared_kv
    out = causal_attention(q, k, v, m["scale"], m.get("softcap"))
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(n, H * dv) * gate) @ w["o"].T, (k, v)


def decayed_outer_products(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: List[float],
                           state: Optional[torch.Tensor] = None):
    """q, k [n, H, d], v [n, H, dv] (after their activation).  S <- decay_h S + k v^T; o = S^T q, token by token.
    -> (o [n, H, dv], final state [H, d, dv])."""
    n, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        for a in range(H):
            S[a] = decay[a] * S[a] + torch.outer(k[t, a], v[t, a])
            out[t, a] = S[a].T @ q[t, a]
    return out, S


def lightning_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d = m["heads"], m["dim"]
    dv = m.get("vdim", d)
    silu = torch.nn.functional.silu
    out, _ = decayed_outer_products(silu(h @ w["q"].T).view(n, H, d), silu(h @ w["k"].T).view(n, H, d),
                                    silu(h @ w["v"].T).view(n, H, dv), m["decay"])
    o = plain_norm(out.reshape(n, H * dv), w["norm"], eps)
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    limit = mlp.get("limit", math.inf)
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def relu2_expert(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ up.T).pow(2) @ down.T


def route(h: torch.Tensor, w: Dict[str, torch.Tensor], router: dict):
    """One token.  -> (chosen experts, their weights)."""
    E, top = router["experts"], router["top"]
    s = torch.sigmoid(w["router"] @ h)
    choice = s + w["correction"] if "correction" in w else s.clone()
    groups = router.get("groups")
    if groups:
        size = E // groups["count"]
        score = [choice[i * size:(i + 1) * size].topk(min(2, size)).values.sum().item() for i in range(groups["count"])]
        best = sorted(range(groups["count"]), key=lambda i: (-score[i], i))[:groups["keep"]]
        allowed = torch.zeros(E, dtype=torch.bool)
        for i in best:
            allowed[i * size:(i + 1) * size] = True
        choice = torch.where(allowed, choice, torch.full_like(choice, -math.inf))
    chosen = sorted(range(E), key=lambda e: (-choice[e].item(), e))[:top]
    weights = s[chosen]
    weights = weights / (weights.sum() + 1e-20) * router.get("scale", 1.0)
    return chosen, weights


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        chosen, weights = route(h[t], w, mlp["router"])
        for e, weight in zip(chosen, weights):
            out[t] += weight * relu2_expert(h[t], w[f"e{e}.up"], w[f"e{e}.down"])
    if mlp.get("shared"):
        out += relu2_expert(h, w["shared.up"], w["shared.down"])
    return out


def _sub(sd: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in sd.items() if k.startswith(prefix)}


def logits(cfg: dict, sd: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None,
           dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Logits [n, vocab] of a whole sequence under weights ``sd`` (checkpoint names), computed in ``dtype``."""
    eps = cfg["norm"]["eps"]
    embed = sd["embed"].to(dtype)
    x = embed[torch.tensor(tokens)]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        h = offset_norm(x, sd[f"l{i}.norm1"].to(dtype), eps)
        w, m = _sub(sd, f"l{i}.mix.", dtype), layer["mixer"]
        if layer["type"] == "attention":
            src = m.get("kv_from")
            y, kept[i] = attention_mixer(h, w, m, kept[src] if src is not None else None)
        elif layer["type"] == "lightning":
            y = lightning_mixer(h, w, m, eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            wm = _sub(sd, f"l{i}.mlp.", dtype)
            y = y + (dense_ff(h, wm, mlp) if mlp["kind"] == "dense" else moe_ff(h, wm, mlp))
        x = x + y
        if residuals is not None:
            residuals.append(x.clone())
    return offset_norm(x, sd["final.norm"].to(dtype), eps) @ embed.T
