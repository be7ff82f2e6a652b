"""Lapilorn: a decoder whose layers are listed one by one in its config.json and whose two sublayers run side by
side on ONE norm of the residual stream.

Each entry of ``layers`` names the layer's token mixer -- ``attention`` (grouped query heads, partial rotary
embedding on neighbouring pairs with long waves slowed down, soft-capped scores, a sigmoid gate on the heads'
output, optionally reading the rotated keys / values of an earlier layer) or ``lightning`` (linear attention with
a constant decay per head and a per-sequence fp32 state) -- with the mixer's sizes, and its feed-forward: ``dense``
(a clamped gated unit), ``moe`` (sigmoid router with group-limited choice, relu^2 experts, an optional shared
expert) or none.

A layer:  h = N(x);  x <- x + (mixer(h) + ff(h)),  N(x) = x / rms(x) * (1 + w).  The stream is fp32; the add of a
layer and the norm of the next one are one kernel.  The logits reuse the embedding table.
Steps arrive in the ragged layout (``InputMetadata.ragged``): any mix of prompt portions and decoded tokens.

Per layer the worker allocates what ``cache_layout`` asks for: pages of keys / values for an attention layer
that owns them, per-sequence state slots for a lightning layer.
"""
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from ..input_metadata import InputMetadata
from ..layers.attention import CappedGatedAttention
from ..layers.basic import ClampedGLU, OffsetRMSNorm, scaled_rotary_frequencies
from ..layers.linear import LinearMethodBase, MergedColumnParallelLinear, RowParallelLinear
from ..layers.moe import GroupRoutedExperts
from ..layers.recurrent import LightningMixer
from ..layers.sampler import Sampler, SamplingMetadata
from ..layers.vocab_parallel_embedding import VocabParallelEmbedding
from ..parallel_state import get_tensor_model_parallel_world_size

_GLU_ALPHA = 1.702                  # the dense feed-forward's gate is g * sigmoid(1.702 g)


def normalize_config(raw: dict) -> dict:
    """The engine's generic geometry keys for a Lapilorn config.json."""
    cfg = dict(raw)
    cfg["architecture"] = "lapilorn"
    cfg["vocab_size"] = raw["vocab"]
    cfg["hidden_size"] = raw["width"]
    cfg["num_hidden_layers"] = len(raw["layers"])
    attn = [l["mixer"] for l in raw["layers"] if l["type"] == "attention"]
    cfg["num_attention_heads"] = attn[0]["heads"] if attn else 1
    cfg["num_key_value_heads"] = attn[0].get("kv_heads", attn[0]["heads"]) if attn else 1
    cfg.setdefault("max_position_embeddings", 1 << 20)       # angles come from fp32 positions: no table to outgrow
    cfg.setdefault("torch_dtype", "bfloat16")
    return cfg


def _shares_kv(m: dict) -> bool:
    return m.get("kv_from") is not None


class LapilornAttention(nn.Module):
    def __init__(self, width: int, m: dict, dtype, linear_method) -> None:
        super().__init__()
        self.shares_kv = _shares_kv(m)
        h, d = m["heads"], m["dim"]
        g, dv = m.get("kv_heads", h), m.get("vdim", d)
        self.q_size, self.k_size, self.v_size, self.o_size = h * d, g * d, g * dv, h * dv
        # q | gate (| k | v): every projection of the layer's input is one GEMM
        sizes = [self.q_size, self.o_size] + ([] if self.shares_kv else [self.k_size, self.v_size])
        self.in_proj = MergedColumnParallelLinear(width, sizes, False, dtype, linear_method)
        self.o_proj = RowParallelLinear(self.o_size, width, False, dtype, linear_method)
        rot = m.get("rot")
        freqs = scaled_rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling")) if rot else None
        self.attn = CappedGatedAttention(h, g, d, dv, m["scale"], m.get("softcap") or 0.0, freqs,
                                         shares_kv=self.shares_kv)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, cache: List[torch.Tensor],
                md: InputMetadata) -> torch.Tensor:
        proj = self.in_proj(h)
        q, gate = proj[:, :self.q_size], proj[:, self.q_size:self.q_size + self.o_size]
        k = v = None
        if not self.shares_kv:
            lo = self.q_size + self.o_size
            k, v = proj[:, lo:lo + self.k_size], proj[:, lo + self.k_size:]
        return self.o_proj(self.attn(q, k, v, gate, positions, cache[0], cache[1], md))

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        parts = [w["q"], w["g"]] + ([] if self.shares_kv else [w["k"], w["v"]])
        self.in_proj.weight.data.copy_(torch.cat(parts, 0))
        self.o_proj.weight.data.copy_(w["o"])


class ClampedGatedMLP(nn.Module):
    """down(g * sigmoid(alpha g) * (u + 1)) with g = min(gate x, limit), u = clamp(up x, -limit, limit)."""

    def __init__(self, width: int, ff: int, limit: float, dtype, linear_method) -> None:
        super().__init__()
        self.gate_up = MergedColumnParallelLinear(width, [ff, ff], False, dtype, linear_method)
        self.down = RowParallelLinear(ff, width, False, dtype, linear_method)
        self.act = ClampedGLU(_GLU_ALPHA, limit, 1.0)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(self.act(self.gate_up(h)))

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        self.gate_up.weight.data.copy_(torch.cat([w["gate"], w["up"]], 0))
        self.down.weight.data.copy_(w["down"])


class LapilornLayer(nn.Module):
    def __init__(self, cfg: dict, index: int, dtype, linear_method) -> None:
        super().__init__()
        layer = cfg["layers"][index]
        width, eps, m = cfg["width"], cfg["norm"]["eps"], layer["mixer"]
        self.kind = layer["type"]
        if self.kind == "attention":
            self.mix = LapilornAttention(width, m, dtype, linear_method)
        elif self.kind == "lightning":
            self.mix = LightningMixer(width, m["heads"], m["dim"], m.get("vdim", m["dim"]), m["decay"], eps, dtype,
                                      linear_method)
        else:
            raise ValueError(f"layer {index}: unknown mixer type {self.kind!r}")
        self.norm1 = OffsetRMSNorm(width, eps, 1.0)
        mlp = layer.get("mlp")
        self.mlp, self.mlp_kind = None, None
        if mlp is not None:
            self.mlp_kind = mlp["kind"]
            if self.mlp_kind == "dense":
                self.mlp = ClampedGatedMLP(width, mlp["ff"], mlp.get("limit", float("inf")), dtype, linear_method)
            elif self.mlp_kind == "moe":
                router, shared = mlp["router"], mlp.get("shared")
                groups = router.get("groups") or {"count": 1, "keep": 1}
                self.mlp = GroupRoutedExperts(width, router["experts"], router["top"], mlp["expert"]["ff"],
                                              shared["ff"] if shared else None, groups["count"], groups["keep"],
                                              router.get("scale", 1.0), dtype, linear_method)
            else:
                raise ValueError(f"layer {index}: unknown feed-forward kind {self.mlp_kind!r}")

    def forward(self, h: torch.Tensor, positions: torch.Tensor, cache: List[torch.Tensor], md: InputMetadata):
        """h: the layer's norm of the stream.  -> the addends of the stream: (mixer output, feed-forward output in
        the activation dtype or None, feed-forward output in fp32 or None)."""
        if self.kind == "attention":
            a = self.mix(h, positions, cache, md)
        else:
            a = self.mix(h, cache, md)
        if self.mlp is None:
            return a, None, None
        if self.mlp_kind == "dense":
            return a, self.mlp(h), None
        shared, routed = self.mlp(h)
        return a, shared, routed


class LapilornForCausalLM(nn.Module):
    uses_ragged_steps = True            # the runner lays every step out as a ragged batch
    supports_float32 = True

    def __init__(self, cfg: dict, dtype: torch.dtype, linear_method: Optional[LinearMethodBase] = None) -> None:
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Lapilorn layers keep a per-sequence state on one GPU: tensor parallelism is "
                                      "not built for them")
        if linear_method is not None:
            raise NotImplementedError("Lapilorn checkpoints are dense: no quantised linear method")
        self.config, self.dtype = cfg, dtype
        self.embed_tokens = VocabParallelEmbedding(cfg["vocab"], cfg["width"], dtype)
        self.layers = nn.ModuleList([LapilornLayer(cfg, i, dtype, None) for i in range(len(cfg["layers"]))])
        self.norm = OffsetRMSNorm(cfg["width"], cfg["norm"]["eps"], 1.0)
        self.sampler = Sampler(cfg["vocab"])
        # set by a caller that wants the stream after every layer (a debugging aid; costs a copy per layer)
        self.keep_residuals: Optional[list] = None

    # ------------------------------------------------------------------ caches
    @staticmethod
    def cache_layout(cfg: dict, block_size: int) -> List[dict]:
        """Per layer: {"paged": [shape per page, ...]} for an attention layer that owns its keys / values,
        {"alias": j} for one that reads layer j's, {"state": [shape per slot, ...]} for a lightning layer
        (state tensors are fp32, paged ones have the model's dtype)."""
        out = []
        for i, layer in enumerate(cfg["layers"]):
            m = layer["mixer"]
            if layer["type"] == "attention":
                src = m.get("kv_from")
                if src is not None:
                    if not (0 <= src < i) or cfg["layers"][src]["type"] != "attention" \
                            or _shares_kv(cfg["layers"][src]["mixer"]):
                        raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
                    out.append({"alias": src})
                else:
                    g = m.get("kv_heads", m["heads"])
                    out.append({"paged": [(block_size, g * m["dim"]), (block_size, g * m.get("vdim", m["dim"]))]})
            elif layer["type"] == "lightning":
                out.append({"state": [(m["heads"], m["dim"], m.get("vdim", m["dim"]))]})
            else:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
        return out

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids, positions, kv_caches, input_metadata: InputMetadata):
        if input_metadata.ragged is None:
            raise RuntimeError("Lapilorn steps need the ragged layout (InputMetadata.ragged)")
        positions = positions.reshape(-1)
        x = self.embed_tokens(input_ids).float()
        h = self.layers[0].norm1(x, self.dtype) if len(self.layers) else None
        for i, layer in enumerate(self.layers):
            a, b, c = layer(h, positions, kv_caches[i], input_metadata)
            nxt = self.layers[i + 1].norm1 if i + 1 < len(self.layers) else self.norm
            h = nxt.add_norm(x, self.dtype, a, b, c)         # x += a + b + c;  h = the next norm of x
            if self.keep_residuals is not None:
                self.keep_residuals.append(x.clone())
        if h is None:
            h = self.norm(x, self.dtype)
        return h

    def sample(self, hidden_states, sampling_metadata: SamplingMetadata):
        return self.sampler(self.embed_tokens.weight, hidden_states, sampling_metadata)

    def compute_logits(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of the given rows of ``forward``'s result: products accumulated and kept in fp32."""
        w = self.embed_tokens.weight
        out = torch.empty(hidden_rows.shape[0], w.shape[0], dtype=torch.float32, device=hidden_rows.device)
        rows32 = hidden_rows.float()
        step = 1 << 14                                        # bounds the fp32 copy of the table's slice
        for lo in range(0, w.shape[0], step):
            out[:, lo:lo + step] = torch.matmul(rows32, w[lo:lo + step].float().t())
        return out

    # ----------------------------------------------------------------- weights
    @torch.no_grad()
    def finish_random_init(self, seed: int) -> None:
        """After the loader's generic random values (no checkpoint): norm weights around zero, routers and
        selection biases of a working model's size."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for layer in self.layers:
            layer.norm1.weight.data.copy_(0.1 * torch.randn(layer.norm1.weight.shape, generator=g))
            if isinstance(layer.mix, LightningMixer):
                layer.mix.out_norm.data.fill_(1.0)
            if isinstance(layer.mlp, GroupRoutedExperts):
                layer.mlp.router.data.copy_(torch.randn(layer.mlp.router.shape, generator=g) * layer.mlp.width ** -0.5)
                layer.mlp.correction.data.copy_(0.1 * torch.randn(layer.mlp.correction.shape, generator=g))
        self.norm.weight.data.zero_()

    def load_weights(self, state: Dict[str, torch.Tensor]) -> None:
        """``state``: checkpoint tensors by name ('embed', 'l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1', 'final.norm')."""
        def cast(t):
            return t.to(self.dtype) if t.dtype.is_floating_point else t
        self.embed_tokens.weight.data.copy_(cast(state["embed"]))
        self.norm.weight.data.copy_(state["final.norm"].float())
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            # routers, selection biases and norm weights stay as stored: their layers keep them in fp32
            layer.mix.load_named({k[len(pre) + 4:]: cast(v) for k, v in state.items() if k.startswith(pre + "mix.")})
            layer.norm1.weight.data.copy_(state[pre + "norm1"].float())
            if layer.mlp is not None:
                layer.mlp.load_named({k[len(pre) + 4:]: (v if k.endswith(("router", "correction")) else cast(v))
                                      for k, v in state.items() if k.startswith(pre + "mlp.")})
