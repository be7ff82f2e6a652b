"""Nepevik: a decoder whose layers are listed one by one in its config.json.

Each entry of ``layers`` names the layer's token mixer -- ``attention`` (sliding window plus kept first
tokens, heads' weights mixed after the softmax, optionally reading the keys / values of an earlier layer),
``channel_delta`` or ``general_delta`` (delta-rule recurrences) -- with the mixer's sizes, and its
feed-forward (experts chosen by a table over token ids, plus a gated shared expert) or none.

A layer adds the NORMED OUTPUT of each sublayer to the residual stream:  x += N(mixer(x));  x += N(ff(x)),
N an RMS norm with a single gain.  The stream is fp32; sublayers read it cast to the model's dtype.
Steps arrive in the ragged layout (``InputMetadata.ragged``): any mix of prompt portions and decoded tokens.

Per layer the worker allocates what ``cache_layout`` asks for: pages of keys / values for an attention layer
that owns them, per-sequence state slots for a recurrent layer.
"""
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from ..input_metadata import InputMetadata
from ..layers.attention import WindowTalkingAttention
from ..layers.basic import ScalarRMSNorm
from ..layers.linear import LinearMethodBase, MergedColumnParallelLinear, RowParallelLinear
from ..layers.moe import TableRoutedExperts
from ..layers.recurrent import ChannelDeltaMixer, GeneralDeltaMixer
from ..layers.sampler import Sampler, SamplingMetadata
from ..layers.vocab_parallel_embedding import ParallelLMHead, VocabParallelEmbedding
from ..parallel_state import get_tensor_model_parallel_world_size

# ranks of the low-rank maps when a config does not give them (a checkpoint's tensor shapes do)
_DEFAULT_RANK = 16


def normalize_config(raw: dict) -> dict:
    """The engine's generic geometry keys for a Nepevik config.json."""
    cfg = dict(raw)
    cfg["architecture"] = "nepevik"
    cfg["vocab_size"] = raw["vocab"]
    cfg["hidden_size"] = raw["width"]
    cfg["num_hidden_layers"] = len(raw["layers"])
    attn = [l["mixer"] for l in raw["layers"] if l["type"] == "attention"]
    cfg["num_attention_heads"] = attn[0]["heads"] if attn else 1
    cfg["num_key_value_heads"] = attn[0]["kv_heads"] if attn else 1
    cfg.setdefault("max_position_embeddings", 1 << 20)       # positions enter nothing: no limit of the model's own
    cfg.setdefault("torch_dtype", "bfloat16")
    return cfg


def _ranks(cfg: dict, index: int) -> Dict[str, int]:
    """Low-rank sizes of layer ``index``: from the checkpoint's shapes when the loader noted them."""
    return cfg.get("_tensor_ranks", {}).get(index, {})


class NepevikAttention(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, dtype, linear_method) -> None:
        super().__init__()
        self.shares_kv = "kv_from" in m and m["kv_from"] is not None
        h, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        self.q_size, self.k_size, self.v_size = h * d, g * d, g * dv
        sizes = [self.q_size] if self.shares_kv else [self.q_size, self.k_size, self.v_size]
        self.in_proj = MergedColumnParallelLinear(width, sizes, False, dtype, linear_method)
        self.o_proj = RowParallelLinear(h * dv, width, False, dtype, linear_method)
        self.attn = WindowTalkingAttention(h, g, d, dv, m["scale"], m["mask"]["size"], m["mask"]["keep_first"], eps,
                                           shares_kv=self.shares_kv)

    def forward(self, h: torch.Tensor, cache: List[torch.Tensor], md: InputMetadata) -> torch.Tensor:
        proj = self.in_proj(h)
        if self.shares_kv:
            out = self.attn(proj, None, None, cache[0], cache[1], md)
        else:
            q, k = proj[:, :self.q_size], proj[:, self.q_size:self.q_size + self.k_size]
            out = self.attn(q, k, proj[:, self.q_size + self.k_size:], cache[0], cache[1], md)
        return self.o_proj(out)

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        parts = [w["q"]] if self.shares_kv else [w["q"], w["k"], w["v"]]
        self.in_proj.weight.data.copy_(torch.cat(parts, 0))
        self.o_proj.weight.data.copy_(w["o"])
        self.attn.q_norm.data.copy_(w["q.norm"].float())
        if not self.shares_kv:
            self.attn.k_norm.data.copy_(w["k.norm"].float())
        self.attn.talk.data.copy_(w["talk"].float())


class NepevikLayer(nn.Module):
    def __init__(self, cfg: dict, index: int, dtype, linear_method) -> None:
        super().__init__()
        layer = cfg["layers"][index]
        width, eps, m = cfg["width"], cfg["norm"]["eps"], layer["mixer"]
        self.kind = layer["type"]
        ranks = _ranks(cfg, index)
        if self.kind == "attention":
            self.mix = NepevikAttention(width, m, eps, dtype, linear_method)
        elif self.kind == "channel_delta":
            self.mix = ChannelDeltaMixer(width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"],
                                         ranks.get("a1", _DEFAULT_RANK), ranks.get("g1", _DEFAULT_RANK), eps, dtype,
                                         linear_method)
        elif self.kind == "general_delta":
            self.mix = GeneralDeltaMixer(width, m["heads"], m["dim"], ranks.get("w1", _DEFAULT_RANK), eps, dtype,
                                         linear_method)
        else:
            raise ValueError(f"layer {index}: unknown mixer type {self.kind!r}")
        self.norm1 = ScalarRMSNorm(eps)
        mlp = layer.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {index}: unknown feed-forward kind {mlp.get('kind')!r}")
            shared = mlp.get("shared")
            self.mlp = TableRoutedExperts(width, cfg["vocab"], mlp["router"]["experts"], mlp["router"]["top"],
                                          mlp["expert"]["ff"], shared["ff"] if shared else None, dtype, linear_method)
            self.norm2 = ScalarRMSNorm(eps)

    def forward(self, x: torch.Tensor, h: torch.Tensor, token_ids: torch.Tensor, cache: List[torch.Tensor],
                md: InputMetadata) -> torch.Tensor:
        """x: the fp32 stream (updated in place); h: x in the activation dtype.  -> the new h."""
        y = self.mix(h, cache, md)
        h = torch.empty_like(h)
        self.norm1.add_to(x, y, cast_out=h)
        if self.mlp is not None:
            y = self.mlp(h, token_ids)
            h = torch.empty_like(h)
            self.norm2.add_to(x, y, cast_out=h)
        return h


class NepevikForCausalLM(nn.Module):
    uses_ragged_steps = True            # the runner lays every step out as a ragged batch
    supports_float32 = True

    def __init__(self, cfg: dict, dtype: torch.dtype, linear_method: Optional[LinearMethodBase] = None) -> None:
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Nepevik layers keep a per-sequence state on one GPU: tensor parallelism is "
                                      "not built for them")
        if linear_method is not None:
            raise NotImplementedError("Nepevik checkpoints are dense: no quantised linear method")
        self.config, self.dtype = cfg, dtype
        self.embed_tokens = VocabParallelEmbedding(cfg["vocab"], cfg["width"], dtype)
        self.layers = nn.ModuleList([NepevikLayer(cfg, i, dtype, None) for i in range(len(cfg["layers"]))])
        self.norm = ScalarRMSNorm(cfg["norm"]["eps"])
        self.lm_head = ParallelLMHead(cfg["vocab"], cfg["width"], dtype)
        self.sampler = Sampler(cfg["vocab"])
        # set by a caller that wants the stream after every layer (a debugging aid; costs a copy per layer)
        self.keep_residuals: Optional[list] = None

    # ------------------------------------------------------------------ caches
    @staticmethod
    def cache_layout(cfg: dict, block_size: int) -> List[dict]:
        """Per layer: {"paged": [shape per page, ...]} for an attention layer that owns its keys / values,
        {"alias": j} for one that reads layer j's, {"state": [shape per slot, ...]} for a recurrent layer
        (state tensors are fp32, paged ones have the model's dtype)."""
        out = []
        for i, layer in enumerate(cfg["layers"]):
            m = layer["mixer"]
            if layer["type"] == "attention":
                src = m.get("kv_from")
                if src is not None:
                    if not (0 <= src < i) or cfg["layers"][src]["type"] != "attention" \
                            or cfg["layers"][src]["mixer"].get("kv_from") is not None:
                        raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
                    out.append({"alias": src})
                else:
                    out.append({"paged": [(block_size, m["kv_heads"] * m["dim"]),
                                          (block_size, m["kv_heads"] * m["vdim"])]})
            elif layer["type"] == "channel_delta":
                channels = 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"]
                out.append({"state": [(m["conv"] - 1, channels), (m["heads"], m["dim"], m["vdim"])]})
            elif layer["type"] == "general_delta":
                out.append({"state": [(m["heads"], m["dim"], m["dim"])]})
            else:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
        return out

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids, positions, kv_caches, input_metadata: InputMetadata):
        del positions                       # no layer of this design rotates or offsets by position
        if input_metadata.ragged is None:
            raise RuntimeError("Nepevik steps need the ragged layout (InputMetadata.ragged)")
        h = self.embed_tokens(input_ids)
        x = h.float()
        for i, layer in enumerate(self.layers):
            h = layer(x, h, input_ids, kv_caches[i], input_metadata)
            if self.keep_residuals is not None:
                self.keep_residuals.append(x.clone())
        return self.norm(x, self.dtype)

    def sample(self, hidden_states, sampling_metadata: SamplingMetadata):
        return self.sampler(self.lm_head.weight, hidden_states, sampling_metadata)

    def compute_logits(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of the given rows of ``forward``'s result."""
        return torch.matmul(hidden_rows, self.lm_head.weight.t()).float()

    # ----------------------------------------------------------------- weights
    @torch.no_grad()
    def finish_random_init(self, seed: int) -> None:
        """After the loader's generic random values (no checkpoint): the tables must name real experts, the
        gains and mixing matrices get values of a working model's size."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for layer in self.layers:
            layer.norm1.weight.data.fill_(1.0)
            if layer.mlp is not None:
                layer.norm2.weight.data.fill_(1.0)
                mlp = layer.mlp
                vocab = mlp.table.shape[0]
                picks = torch.rand(vocab, mlp.num_experts, generator=g).argsort(dim=1)[:, :mlp.top]
                mlp.table.data.copy_(picks.to(torch.int32))
            mix = layer.mix
            if isinstance(mix, NepevikAttention):
                heads = mix.attn.heads
                mix.attn.talk.data.copy_(torch.eye(heads) + 0.1 * torch.randn(heads, heads, generator=g))
                mix.attn.q_norm.data.fill_(1.0)
                if mix.attn.k_norm is not None:
                    mix.attn.k_norm.data.fill_(1.0)
            else:
                mix.out_norm.data.fill_(1.0)
                if isinstance(mix, ChannelDeltaMixer):
                    mix.conv_taps.data.copy_(0.5 * torch.randn(mix.conv_taps.shape, generator=g))
        self.norm.weight.data.fill_(1.0)

    @staticmethod
    def note_tensor_shapes(cfg: dict, shapes: Dict[str, tuple]) -> None:
        """Sizes that only the checkpoint's tensor shapes give (the ranks of the low-rank maps)."""
        ranks: Dict[int, Dict[str, int]] = {}
        for name, shape in shapes.items():
            parts = name.split(".")
            if len(parts) == 3 and parts[1] == "mix" and parts[2] in ("a1", "g1", "w1") and parts[0][1:].isdigit():
                ranks.setdefault(int(parts[0][1:]), {})[parts[2]] = shape[0]
        cfg["_tensor_ranks"] = ranks

    def load_weights(self, state: Dict[str, torch.Tensor]) -> None:
        """``state``: checkpoint tensors by name ('embed', 'l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1', 'final.norm',
        'head')."""
        def cast(t):
            return t.to(self.dtype) if t.dtype.is_floating_point else t
        self.embed_tokens.weight.data.copy_(cast(state["embed"]))
        self.lm_head.weight.data.copy_(cast(state["head"]))
        self.norm.weight.data.copy_(state["final.norm"].float().reshape(1))
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            layer.mix.load_named({k[len(pre) + 4:]: cast(v) for k, v in state.items() if k.startswith(pre + "mix.")})
            layer.norm1.weight.data.copy_(state[pre + "norm1"].float().reshape(1))
            if layer.mlp is not None:
                layer.mlp.load_named({k[len(pre) + 4:]: cast(v) for k, v in state.items()
                                      if k.startswith(pre + "mlp.")})
                layer.norm2.weight.data.copy_(state[pre + "norm2"].float().reshape(1))
