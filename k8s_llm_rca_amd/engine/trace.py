"""Replay of a recorded schedule through the engine: given token ids step by
step, logits out, nothing sampled.

Steps arrive as JSON lines ``{"step": n, "entries": [{"id", "tokens", "want"}],
"end": [ids]}``: every entry brings a request's next tokens (a request is
admitted at its first entry and may skip steps), ``want`` the offsets among them
whose logits are written, ``end`` the requests whose pages and state go back to
the pools after the step.  All entries of a step are ONE engine step
(:meth:`LLMEngine.feed`): portions of prompts beside single decoded tokens.
For a step with wanted rows ``<out>/<step>.f32`` holds them as little-endian
fp32 [wanted, vocab]; after every step ``done <step>`` is printed.
"""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, IO, Optional

import numpy as np
import torch

from .engine import EngineConfig, LLMEngine


def make_engine(model_dir: str, dtype: torch.dtype, max_tokens: int, device: Optional[str] = None,
                state_slots: int = 4, block_size: int = 64) -> LLMEngine:
    """An engine over the checkpoint in ``model_dir`` whose page pool holds ``max_tokens`` tokens
    (each live request rounded up to whole pages) and ``state_slots`` sequences' state."""
    if device is None:
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: the replay runs the HIP kernels (pass --device cpu for the reference ops)")
        device = "cuda"
    if device.startswith("cuda"):
        torch.backends.cuda.matmul.allow_tf32 = False   # float32 means float32
        torch.backends.cudnn.allow_tf32 = False
    nb = max(1, -(-int(max_tokens) // block_size))
    cfg = EngineConfig(weights=model_dir, device=device, dtype=dtype, num_blocks=nb, block_size=block_size,
                       max_batch_tokens=max(8192, nb * block_size), max_context=nb * block_size,
                       state_slots=state_slots, use_graphs=False, prefix_sharing=False, kv_host_gb=0.0)
    return LLMEngine(cfg)


def replay(eng: LLMEngine, lines: IO[str], out_dir: str, log: IO[str] = sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    sid_of: Dict[str, int] = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = []
        n_want = 0
        for e in st.get("entries", []):
            rid = str(e["id"])
            if rid not in sid_of:
                sid_of[rid] = eng.new_sequence()
            want = [int(w) for w in e.get("want", [])]
            n_want += len(want)
            entries.append((sid_of[rid], [int(t) for t in e["tokens"]], want))
        if entries:
            logits = eng.feed(entries)
            if n_want:
                arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4", copy=False)
                assert arr.shape[0] == n_want
                tmp = os.path.join(out_dir, f".{st['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(np.ascontiguousarray(arr).tobytes())
                os.replace(tmp, os.path.join(out_dir, f"{st['step']}.f32"))
            elif eng.device.type == "cuda":
                torch.cuda.synchronize(eng.device)
        for rid in st.get("end", []):
            sid = sid_of.pop(str(rid), None)
            if sid is not None:
                eng.release_sequence(sid)
        log.write(f"done {st['step']}\n")
        log.flush()
    return 0


def main(model_dir: str, dtype_name: str, out_dir: str, max_tokens: int, device: Optional[str] = None) -> int:
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype_name]
    eng = make_engine(model_dir, dtype, max_tokens, device)
    return replay(eng, sys.stdin, out_dir)
