"""Small random Lapilorn models on disk.  The engine harness (``Replayer``, ``make_engine``, ``write_model``,
``row_error``) is the one of ``nepevik_util``: it only speaks to the engine."""
from typing import Dict, List, Optional

import torch

from nepevik_util import Replayer, make_engine, row_error, write_model  # noqa: F401  (re-exported)


def attention(heads=4, kv_heads=2, dim=16, vdim=32, scale=0.3, softcap=6.0, rot_dims=8, base=50.0, scaling=None,
              kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
         "rot": {"base": base, "dims": rot_dims}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def lightning(heads=3, dim=24, vdim=16, decay=(0.5, 0.9, 0.99)):
    assert len(decay) == heads
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def dense(ff=40, limit=0.8):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=6, top=2, ff=24, shared_ff=40, groups=3, keep=2, scale=1.3):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups:
        router["groups"] = {"count": groups, "keep": keep}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared_ff:
        out["shared"] = {"ff": shared_ff}
    return out


def config(layers: List[dict], mlps: List[Optional[dict]], vocab=97, width=48, eps=1e-5) -> dict:
    out = []
    for layer, mlp in zip(layers, mlps):
        entry = dict(layer)
        entry["mlp"] = mlp
        out.append(entry)
    return {"architecture": "Lapilorn", "layers": out, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bf16 weights under the checkpoint's names; magnitudes chosen so that every mechanism matters: scores that
    reach the cap, gates and up-projections beyond the limit, selection biases that change the choice (some
    choice scores negative), norm weights away from zero."""
    g = torch.Generator().manual_seed(seed)
    width, vocab = cfg["width"], cfg["vocab"]

    def rnd(*shape, scale=1.0):
        return (torch.randn(tuple(shape), generator=g) * scale).to(torch.bfloat16)

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, scale=gain / inp ** 0.5)

    sd = {"embed": rnd(vocab, width), "final.norm": rnd(width, scale=0.2)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        sd[p + "norm1"] = rnd(width, scale=0.2)
        h, d = m["heads"], m["dim"]
        dv = m.get("vdim", d)
        if layer["type"] == "attention":
            kv = m.get("kv_heads", h)
            sd[p + "mix.q"] = lin(h * d, width, 3.0)
            if m.get("kv_from") is None:
                sd[p + "mix.k"] = lin(kv * d, width, 3.0)
                sd[p + "mix.v"] = lin(kv * dv, width)
        else:
            sd[p + "mix.q"], sd[p + "mix.k"] = lin(h * d, width, 1.5), lin(h * d, width, 1.5)
            sd[p + "mix.v"] = lin(h * dv, width, 1.5)
            sd[p + "mix.norm"] = rnd(h * dv, scale=0.3) + 1.0
        sd[p + "mix.g"] = lin(h * dv, width, 2.0)
        sd[p + "mix.o"] = lin(width, h * dv)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            sd[p + "mlp.gate"], sd[p + "mlp.up"] = lin(mlp["ff"], width, 1.5), lin(mlp["ff"], width, 1.5)
            sd[p + "mlp.down"] = lin(width, mlp["ff"])
        else:
            e, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for j in range(e):
                sd[p + f"mlp.e{j}.up"], sd[p + f"mlp.e{j}.down"] = lin(ff, width, 2.0), lin(width, ff, 1.0)
            sd[p + "mlp.router"] = lin(e, width, 2.0)
            sd[p + "mlp.correction"] = rnd(e, scale=0.5) - 0.4
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                sd[p + "mlp.shared.up"], sd[p + "mlp.shared.down"] = lin(sf, width, 2.0), lin(width, sf, 1.0)
    return sd
