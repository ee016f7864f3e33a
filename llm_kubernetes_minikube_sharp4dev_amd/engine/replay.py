"""Trace replay: feed given token ids through a model step by step and write logits.

Nothing is sampled.  Each input line is one engine step -- for every request its next tokens (a
whole prompt, a portion of one, or a single token) and the places among them whose logits are
wanted -- and all entries of a line run as ONE batch through ``LLMEngine.replay_step``: the model
runner, paged cache, state slots and kernels that generation uses.  The cache pool is sized for
``max_tokens`` live tokens and ``max_seqs`` live requests, so finished requests' pages and slots
are handed out again.

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}

For a step that wants something, ``<out>/<step>.f32`` holds the logits as little-endian f32
[wanted, vocab] in the order of the entries and of ``want``; after every step ``done <step>`` is
printed and flushed.
"""
from __future__ import annotations

import json
import os
import sys

import torch


def build_engine(model_dir: str, dtype: str = "bfloat16", max_tokens: int = 8192, max_seqs: int = 4, block_size: int = 16,
                 device: str = "auto", use_graphs: bool = True):
    from ..models import load_decoder_dir
    from .llm_engine import LLMEngine

    dt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    if device == "auto":
        device = "cuda" if torch.cuda.is_available() else "cpu"
    if dt == torch.float32:  # true 32-bit products in the vendor GEMMs the f32 path uses
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    model = load_decoder_dir(model_dir, device=device, dtype=dt)
    num_blocks = max(1, -(-int(max_tokens) // block_size))
    # no request can be longer than the pool; a design without learned positions names no smaller bound
    max_len = min(int(model.cfg.max_position), num_blocks * block_size)
    return LLMEngine(model, None, block_size=block_size, max_model_len=max_len, max_num_seqs=max_seqs,
                     num_blocks=num_blocks, eos_ids=set(), use_graphs=use_graphs, enable_prefix_caching=True)


def run_trace(model_dir: str, dtype: str, out_dir: str, max_tokens: int, lines=None, out=None, max_seqs: int = 4,
              device: str = "auto", use_graphs: bool = True) -> int:
    lines = sys.stdin if lines is None else lines
    out = sys.stdout if out is None else out
    eng = build_engine(model_dir, dtype, max_tokens, max_seqs, device=device, use_graphs=use_graphs)
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in st.get("entries", [])]
        lg = eng.replay_step(entries, st.get("end", []))
        if lg is not None and lg.shape[0]:
            lg.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4").tofile(
                os.path.join(out_dir, f"{st['step']}.f32"))
        out.write(f"done {st['step']}\n")
        out.flush()
    return 0
