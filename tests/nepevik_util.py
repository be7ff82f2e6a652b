"""Small random Nepevik models on disk and a harness that drives the engine step by step."""
import json
import os
from typing import Dict, List, Optional

import torch


def attention(heads=4, kv_heads=2, dim=16, vdim=32, window=8, keep_first=3, scale=0.25, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "mask": {"size": window, "keep_first": keep_first}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def channel_delta(heads=4, kv_heads=2, dim=16, vdim=32, conv=4):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                               "conv": conv}}


def general_delta(heads=3, dim=24):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}}


def moe(experts=5, top=2, ff=24, shared_ff=40):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared_ff} if shared_ff else None}


def config(layers: List[dict], mlps: List[Optional[dict]], vocab=97, width=48, eps=1e-5) -> dict:
    out = []
    for layer, mlp in zip(layers, mlps):
        entry = dict(layer)
        entry["mlp"] = mlp
        out.append(entry)
    return {"architecture": "Nepevik", "layers": out, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg: dict, seed: int, decay_rank=6, gate_rank=5) -> Dict[str, torch.Tensor]:
    """bf16 weights (int32 tables) under the checkpoint's names; magnitudes chosen so that every mechanism
    matters: decays well inside (0, 1), gates and removal rates spread, norms' gains away from 1."""
    g = torch.Generator().manual_seed(seed)
    width, vocab = cfg["width"], cfg["vocab"]

    def rnd(*shape, scale=1.0):
        return (torch.randn(tuple(shape), generator=g) * scale).to(torch.bfloat16)

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, scale=gain / inp ** 0.5)

    sd = {"embed": rnd(vocab, width), "head": lin(vocab, width), "final.norm": rnd(scale=0.2) + 1.0}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        sd[p + "norm1"] = rnd(scale=0.2) + 1.0
        if layer["type"] == "attention":
            h, kv, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd[p + "mix.q"] = lin(h * d, width, 2.0)
            sd[p + "mix.q.norm"] = rnd(h * d, scale=0.3) + 1.0
            if m.get("kv_from") is None:
                sd[p + "mix.k"] = lin(kv * d, width, 2.0)
                sd[p + "mix.v"] = lin(kv * dv, width)
                sd[p + "mix.k.norm"] = rnd(kv * d, scale=0.3) + 1.0
            sd[p + "mix.talk"] = (torch.eye(h) + 0.4 * torch.randn(h, h, generator=g)).to(torch.bfloat16)
            sd[p + "mix.o"] = lin(width, h * dv)
        elif layer["type"] == "channel_delta":
            h, kv, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for name, size in (("q", kv * d), ("k", kv * d), ("v", h * dv)):
                sd[p + f"mix.{name}"] = lin(size, width, 2.0)
                sd[p + f"mix.{name}.conv"] = rnd(size, taps, scale=0.6)
            sd[p + "mix.b"] = lin(h, width, 2.0)
            sd[p + "mix.A_log"] = rnd(h, scale=0.5)
            sd[p + "mix.norm"] = rnd(dv, scale=0.3) + 1.0
            sd[p + "mix.a1"], sd[p + "mix.a2"] = lin(decay_rank, width), lin(h * d, decay_rank, 2.0)
            sd[p + "mix.dt_bias"] = rnd(h * d, scale=1.0) - 1.0
            sd[p + "mix.g1"], sd[p + "mix.g2"] = lin(gate_rank, width), lin(h * dv, gate_rank, 2.0)
            sd[p + "mix.o"] = lin(width, h * dv)
        else:
            h, d = m["heads"], m["dim"]
            for name in ("r", "k", "v", "g", "a"):
                sd[p + f"mix.{name}"] = lin(h * d, width, 2.0)
            sd[p + "mix.a.b"] = rnd(h * d, scale=0.5)
            sd[p + "mix.w1"], sd[p + "mix.w2"] = lin(decay_rank, width, 2.0), lin(h * d, decay_rank, 2.0)
            sd[p + "mix.w0"] = rnd(h * d, scale=1.0)
            sd[p + "mix.norm"] = rnd(h * d, scale=0.3) + 1.0
            sd[p + "mix.o"] = lin(width, h * d)
        mlp = layer.get("mlp")
        if mlp is not None:
            sd[p + "norm2"] = rnd(scale=0.2) + 1.0
            e, top, ff = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
            for j in range(e):
                sd[p + f"mlp.e{j}.up"], sd[p + f"mlp.e{j}.down"] = lin(ff, width, 2.0), lin(width, ff, 2.0)
            sd[p + "mlp.table"] = torch.rand(vocab, e, generator=g).argsort(1)[:, :top].to(torch.int32).contiguous()
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                sd[p + "mlp.shared.up"], sd[p + "mlp.shared.down"] = lin(sf, width, 2.0), lin(width, sf, 2.0)
                sd[p + "mlp.shared.sg"] = lin(1, width, 2.0)
    return sd


def write_model(path: str, cfg: dict, sd: Dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    return path


def make_engine(model_dir: str, dtype: str, max_tokens: int = 512, max_requests: int = 4, block_size: int = 16,
                max_num_batched_tokens: Optional[int] = None):
    from splitwise_amd.engine.arg_utils import EngineArgs
    from splitwise_amd.engine.llm_engine import LLMEngine
    torch.backends.cuda.matmul.allow_tf32 = False
    blocks = -(-max_tokens // block_size)
    return LLMEngine.from_engine_args(EngineArgs(
        model=model_dir, dtype=dtype, block_size=block_size, max_model_len=blocks * block_size,
        max_num_seqs=max_requests, max_num_batched_tokens=max_num_batched_tokens or blocks * block_size,
        num_gpu_blocks_override=blocks, swap_space=0, enforce_eager=True))


class Replayer:
    """Feeds given tokens through an engine in steps of the caller's choosing and collects the logits of every
    position: ``step({"a": 5, "b": 1})`` runs the next 5 tokens of request a beside the next one of b."""

    def __init__(self, engine, requests: Dict[str, List[int]]) -> None:
        from splitwise_amd.sampling_params import SamplingParams
        self.engine, self.requests = engine, requests
        self.at = {rid: 0 for rid in requests}
        self.logits = {rid: [None] * len(tokens) for rid, tokens in requests.items()}
        self.params = SamplingParams(temperature=0.0, max_tokens=1)
        self.live = set()

    def step(self, counts: Dict[str, int]) -> None:
        plan, want = {}, {}
        for rid, n in counts.items():
            lo = self.at[rid]
            tokens = self.requests[rid][lo:lo + n]
            assert len(tokens) == n
            if rid in self.live:
                self.engine.extend_request(rid, tokens)
            else:
                self.engine.add_request(rid, None, self.params, prompt_token_ids=list(tokens))
                self.live.add(rid)
            plan[rid], want[rid] = n, list(range(n))
        out = self.engine.step_planned(plan, want)
        for rid, n in counts.items():
            rows = out[rid].float().cpu()
            for k in range(n):
                self.logits[rid][self.at[rid] + k] = rows[k]
            self.at[rid] += n
            if self.at[rid] == len(self.requests[rid]):
                self.end(rid)

    def end(self, rid: str) -> None:
        if rid in self.live:
            self.engine.abort_request([rid])
            self.live.discard(rid)

    def run_alone(self, rid: str, portions: List[int]) -> torch.Tensor:
        for n in portions:
            self.step({rid: n})
        return self.result(rid)

    def result(self, rid: str) -> torch.Tensor:
        return torch.stack(self.logits[rid])


def row_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest per-position error of logits: differences with their mean taken off, root mean square over the
    vocabulary, relative to the spread of the expected logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    scale = (want.double() - want.double().mean(-1, keepdim=True)).pow(2).mean().sqrt()
    return float(d.pow(2).mean(-1).sqrt().max() / scale)
