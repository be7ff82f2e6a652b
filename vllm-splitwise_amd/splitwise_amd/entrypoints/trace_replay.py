"""Replays a recorded schedule: given token ids go through the engine step by step, nothing is sampled, and
the logits at the places a step names are written out.

    python -m splitwise_amd.entrypoints.trace_replay --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object per line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
``entries``: per request its next tokens (a request is admitted at its first entry and may sit out steps) and the
places among them whose logits are wanted; all entries of a step are ONE engine step.  ``end``: requests that
are finished after the step; their blocks and state slot go back to the pools.  For a step that wants logits
``<out>/<step>.f32`` is written (little-endian fp32 [wanted, vocab], in the order of the entries); after every
step ``done <step>`` is printed.

The engine is the one that serves the model: its scheduler places the step (admission, block tables, state
slots), its worker runs it.  The cache pool holds ``--max-tokens`` tokens (rounded up to whole blocks) and
there are ``--max-requests`` state slots, so pages and slots are reused as requests come and go.
"""
import argparse
import json
import os
import sys

# fp32 means fp32 whatever the caller's environment says: these are read when torch (or the BLAS library) loads
for _name in ("TORCH_ALLOW_TF32_CUBLAS_OVERRIDE", "HIPBLASLT_ALLOW_TF32", "ROCBLAS_XF32_XDL_MATH_OP"):
    os.environ.pop(_name, None)

import torch  # noqa: E402


def _ensure_built(architecture_needs_mixers: bool) -> None:
    if not architecture_needs_mixers:
        return
    from .. import _C_mixers
    if not os.path.exists(_C_mixers.library_path()):
        _C_mixers.build_library()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-requests", type=int, default=4)
    ap.add_argument("--block-size", type=int, default=16)
    args = ap.parse_args(argv)

    from ..config import ModelConfig
    from ..engine.arg_utils import EngineArgs
    from ..engine.llm_engine import LLMEngine
    from ..sampling_params import SamplingParams

    probe = ModelConfig(args.model, args.dtype)
    if not probe.uses_ragged_steps:
        print(f"trace replay needs a model that takes ragged steps; {probe.architecture} does not", file=sys.stderr)
        return 3
    _ensure_built(True)
    # fp32 means fp32: no reduced-precision matrix mode
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")

    bs = args.block_size
    blocks = -(-args.max_tokens // bs)
    engine = LLMEngine.from_engine_args(EngineArgs(
        model=args.model, dtype=args.dtype, block_size=bs, max_model_len=blocks * bs, max_num_seqs=args.max_requests,
        max_num_batched_tokens=max(blocks * bs, args.max_requests), num_gpu_blocks_override=blocks, swap_space=0,
        enforce_eager=True))
    vocab = engine.model_config.get_vocab_size()
    params = SamplingParams(temperature=0.0, max_tokens=1)
    os.makedirs(args.out, exist_ok=True)
    live = set()
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        plan, want = {}, {}
        for entry in step["entries"]:
            rid, tokens = str(entry["id"]), [int(t) for t in entry["tokens"]]
            if not tokens:
                continue                                   # nothing to run for this request in this step
            if rid in live:
                engine.extend_request(rid, tokens)
            else:
                engine.add_request(rid, None, params, prompt_token_ids=tokens)
                live.add(rid)
            plan[rid] = len(tokens)
            if entry.get("want"):
                want[rid] = [int(p) for p in entry["want"]]
                if min(want[rid]) < 0 or max(want[rid]) >= len(tokens):
                    raise ValueError(f"step {step['step']}, request {rid}: a wanted place lies outside its tokens")
        if plan:
            logits = engine.step_planned(plan, want)
            if want:
                rows = torch.cat([logits[str(e["id"])] for e in step["entries"] if e.get("want") and e["tokens"]], 0)
                data = rows.float().cpu().numpy().astype("<f4")
                assert data.shape[1] == vocab
                tmp = os.path.join(args.out, f".{step['step']}.part")
                data.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step['step']}.f32"))
        ended = [str(r) for r in step.get("end", []) if str(r) in live]
        if ended:
            engine.abort_request(ended)
            live.difference_update(ended)
        print(f"done {step['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
