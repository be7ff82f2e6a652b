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
    """y [heads, size]: neighbours (2i, 2i + 1) of the first 2 * len(freqs) coordinates turn by position * f_i."""
    out = y.clone()
    for i, f in enumerate(freqs):
        a = torch.tensor(float(position), dtype=torch.float32) * torch.tensor(f, dtype=torch.float32)
        c, s = torch.cos(a), torch.sin(a)
        u, v = y[:, 2 * i], y[:, 2 * i + 1]
        out[:, 2 * i] = u * c - v * s
        out[:, 2 * i + 1] = v * c + u * s
    return out


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, shared_kv=None):
    """-> (output [n, width], (rotated keys, values) as a later layer may reuse them)."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    freqs = rotary_frequencies(m["rot"]) if m.get("rot") else []
    q = (h @ w["q"].T).view(n, H, d)
    q = torch.stack([rotate(q[t], t, freqs) for t in range(n)])
    if shared_kv is None:
        k = (h @ w["k"].T).view(n, G, d)
        k = torch.stack([rotate(k[t], t, freqs) for t in range(n)])
        v = (h @ w["v"].T).view(n, G, dv)
    else:
        k, v = shared_kv
    cap = m.get("softcap")
    out = torch.zeros(n, H, dv)
    for t in range(n):
        for a in range(H):
            g = a // (H // G)
            s = (k[:t + 1, g] @ q[t, a]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            p = torch.softmax(s, 0)
            out[t, a] = p @ v[:t + 1, g]
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(n, H * dv) * gate) @ w["o"].T, (k, v)


def lightning_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q = silu(h @ w["q"].T).view(n, H, d)
    k = silu(h @ w["k"].T).view(n, H, d)
    v = silu(h @ w["v"].T).view(n, H, dv)
    out = torch.zeros(n, H, dv)
    for a in range(H):
        S = torch.zeros(d, dv)
        for t in range(n):
            S = m["decay"][a] * S + torch.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    o = plain_norm(out.reshape(n, H * dv), w["norm"], eps)
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    limit = mlp["limit"]
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def relu2_expert(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ up.T).pow(2) @ down.T


def route(h: torch.Tensor, w: Dict[str, torch.Tensor], router: dict):
    """One token.  -> (chosen experts, their weights)."""
    E, top = router["experts"], router["top"]
    s = torch.sigmoid(w["router"].float() @ h.float())
    choice = s + w["correction"].float() if "correction" in w else s.clone()
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
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0])
    for t in range(h.shape[0]):
        chosen, weights = route(h[t], w, mlp["router"])
        for e, weight in zip(chosen, weights):
            out[t] += weight * relu2_expert(h[t], w[f"e{e}.up"], w[f"e{e}.down"])
    if mlp.get("shared"):
        out += relu2_expert(h, w["shared.up"], w["shared.down"])
    return out


def _sub(sd: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.float() for k, v in sd.items() if k.startswith(prefix)}


def logits(cfg: dict, sd: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None) -> torch.Tensor:
    """fp32 logits [n, vocab] of a whole sequence under weights ``sd`` (checkpoint names)."""
    eps = cfg["norm"]["eps"]
    embed = sd["embed"].float()
    x = embed[torch.tensor(tokens)]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        h = offset_norm(x, sd[f"l{i}.norm1"].float(), eps)
        w, m = _sub(sd, f"l{i}.mix."), layer["mixer"]
        if layer["type"] == "attention":
            src = m.get("kv_from")
            y, kept[i] = attention_mixer(h, w, m, kept[src] if src is not None else None)
        elif layer["type"] == "lightning":
            y = lightning_mixer(h, w, m, eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            wm = _sub(sd, f"l{i}.mlp.")
            y = y + (dense_ff(h, wm, mlp) if mlp["kind"] == "dense" else moe_ff(h, wm, mlp))
        x = x + y
        if residuals is not None:
            residuals.append(x.clone())
    return offset_norm(x, sd["final.norm"].float(), eps) @ embed.T
