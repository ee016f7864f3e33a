"""Lebepel: a hybrid decoder of sigmoid-attention and Mamba-2 layers in parallel blocks.

    x   = embed[token] + pos[position]                         (the "embedding output", f32)
    per layer run:  h = x / rms(x) * (1 + w_norm);  x += m * (mixer(h) + ff(h))
    logits = cap * tanh(head(x / rms(x) * (1 + w_final)) / cap)

A configurable span of layers runs several times with the same weights; every pass has its own
KV cache or recurrent state, and the embedding output is added to the stream once before each
pass after the first.  Mixers: ``models.attention.sigmoid_paged_attention`` (paged K/V) and
``models.ssm.mamba2_mixer`` (per-sequence state slots).

MI355X layout decisions:
  * the residual stream is f32 and never leaves one fused kernel per block: the scaled sum of the
    previous block's two sublayer outputs, the embedding re-injection and the next block's norm
    are a single pass over the row (``ops.stream_rmsnorm``); the final norm runs only on the rows
    that feed the LM head;
  * q | k | v are one projection with its bias in the GEMM epilogue, gate | up one GEMM with the
    SwiGLU epilogue (the framework's MFMA GEMMs; shapes they do not tile go to the vendor library);
  * q / k unit norms and the paged K/V write are one kernel; scores, the distance penalty and the
    sigmoid weights are f32 inside the attention kernels;
  * conv / SSM states live in slot-indexed tensors the engine's state pool hands out, so chunked
    prefill, decode and mixed batches share one code path.

Checkpoint format (``load_checkpoint_dir``): ``config.json`` (``LebepelConfig.from_json``) and
``model.safetensors`` with ``embed``, ``pos``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``; linear weights [out, in].
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops
from ..parallel.tp import SINGLE, TPGroup
from .attention import AttnMeta, SigmoidAttnSpec, sigmoid_paged_attention
from .configs import LebepelConfig, pad_vocab
from .ssm import Mamba2Spec, mamba2_mixer


# The q|k|v bias either rides in the projection GEMM's epilogue (False) or is added in f32 by the
# unit-norm kernel, so that the projection runs on the bias-free decode GEMMs (True).
FUSE_QKV_BIAS = True


class LebepelLayer(nn.Module):
    def __init__(self, cfg: LebepelConfig, spec, dtype, device):
        super().__init__()
        W = cfg.hidden
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)   # small per-head / per-channel constants stay f32

        def P(*shape, **kw):
            return nn.Parameter(torch.zeros(*shape, **kw), requires_grad=False)

        self.type = spec.type
        self.norm1 = P(W, **f)
        if spec.type == "attention":
            t = self.true = SigmoidAttnSpec.from_dict(spec.mixer)   # the checkpoint's sizes
            # head sizes padded to the kernels' 8-element fragments with zero weight rows / columns
            a = self.spec = SigmoidAttnSpec(t.heads, t.kv_heads, -(-t.dim // 8) * 8, -(-t.vdim // 8) * 8, t.scale, t.dim)
            self.qkv, self.qkv_b = P(a.qkv_out, W, **e), P(a.qkv_out, **e)
            self.o, self.o_b = P(W, a.heads * a.vdim, **e), P(W, **f)   # o_b is added in the f32 stream update
            self.r1, self.r2, self.pb = P(a.heads, **f), P(a.heads, **f), P(a.heads, **f)
        else:
            s = self.spec = Mamba2Spec.from_dict(spec.mixer)
            # rows [z | x B C | dt], padded with zero rows to the decode GEMMs' 128-column tiles
            self.in_proj = P(-(-s.proj_out // 128) * 128, W, **e)
            self.conv_w, self.conv_b = P(s.conv_channels, s.conv, **f), P(s.conv_channels, **f)
            self.dt_bias, self.A_log, self.D = P(s.heads, **f), P(s.heads, **f), P(s.heads, **f)
            self.mix_norm = P(s.inner, **f)
            self.o = P(W, s.inner, **e)
        self.ff = int(spec.mlp["ff"]) if spec.mlp else 0
        self.ff_p = -(-self.ff // 8) * 8     # padded with zero gate / up rows and down columns (16-byte rows)
        if self.ff:
            self.gate_up, self.down = P(2 * self.ff_p, W, **e), P(W, self.ff_p, **e)


class LebepelModel(nn.Module):
    stateful = True            # recurrent state per sequence: no prefix reuse, no multi-row decode of one sequence

    def __init__(self, cfg: LebepelConfig, tp: TPGroup = SINGLE, dtype=torch.bfloat16, device="cpu"):
        super().__init__()
        if tp.enabled:
            raise NotImplementedError("the Lebepel decoder runs on one GPU (no tensor-parallel sharding)")
        self.cfg, self.tp, self.dtype, self.device = cfg, tp, dtype, torch.device(device)
        e = dict(dtype=dtype, device=device)
        self.vocab_lo, self.vocab_local = 0, cfg.vocab_size
        self.embed = nn.Parameter(torch.zeros(cfg.vocab_size, cfg.hidden, **e), requires_grad=False)
        self.pos = nn.Parameter(torch.zeros(cfg.max_position, cfg.hidden, **e), requires_grad=False)
        self.layers = nn.ModuleList([LebepelLayer(cfg, l, dtype, device) for l in cfg.layers])
        self.final_norm = nn.Parameter(torch.zeros(cfg.hidden, dtype=torch.float32, device=device), requires_grad=False)
        # head rows padded (zero rows) so that logits rows start 32-byte aligned for the sampling kernels;
        # the padding columns are sliced off before anything reads the logits
        self.lm_head = nn.Parameter(torch.zeros(pad_vocab(cfg.vocab_size, 64), cfg.hidden, **e), requires_grad=False)
        self.runs = cfg.layer_runs()
        self.reinject = any(add for _, add in self.runs)
        # the runner's attention workspaces are sized from these (largest attention layer)
        att = [l.spec for l in self.layers if l.type == "attention"]
        self.hq = max((a.heads for a in att), default=1)
        self.hkv = max((a.kv_heads for a in att), default=1)
        self.D = max((max(a.dim, a.vdim) for a in att), default=16)

    # ------------------------------------------------------------------ weights
    @torch.no_grad()
    def random_init(self, seed: int = 0, std: float = 0.02):
        gen_dev = self.device if self.device.type == "cuda" else torch.device("cpu")

        def rnd(p, i, scale, shift=0.0):
            g = torch.Generator(device=gen_dev).manual_seed(seed * 7919 + i * 104729)
            p.copy_((torch.randn(p.shape, generator=g, device=gen_dev) * scale + shift).to(p.dtype))

        W = self.cfg.hidden
        for i, (name, p) in enumerate(self.named_parameters()):
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "final_norm", "mix_norm"):
                rnd(p, i, 0.05, 1.0 if leaf == "mix_norm" else 0.0)
            elif leaf in ("qkv_b", "o_b", "conv_b", "pb"):
                rnd(p, i, 0.1)
            elif leaf == "r1":
                rnd(p, i, 0.1, 0.5)
            elif leaf == "r2":
                p.copy_((torch.rand(p.shape, device=gen_dev, generator=torch.Generator(device=gen_dev).manual_seed(
                    seed * 7919 + i * 104729)) * 0.5 + 0.05).to(p.dtype))
            elif leaf == "dt_bias":
                rnd(p, i, 0.5, -1.0)
            elif leaf == "A_log":
                rnd(p, i, 0.3, 0.0)
            elif leaf == "D":
                rnd(p, i, 0.2, 1.0)
            elif leaf == "conv_w":
                rnd(p, i, 0.3)
            elif leaf in ("embed", "pos"):
                rnd(p, i, 0.5)
            else:  # projections: unit-variance outputs for unit-variance inputs
                rnd(p, i, 1.0 / math.sqrt(p.shape[1]))
        for L in self.layers:
            if L.type == "attention" and (L.spec.dim != L.true.dim or L.spec.vdim != L.true.vdim):
                a, t = L.spec, L.true
                k = 0
                for h, d, dp in ((a.heads, t.dim, a.dim), (a.kv_heads, t.dim, a.dim), (a.kv_heads, t.vdim, a.vdim)):
                    L.qkv[k:k + h * dp].view(h, dp, -1)[:, d:] = 0
                    L.qkv_b[k:k + h * dp].view(h, dp)[:, d:] = 0
                    k += h * dp
                L.o.view(L.o.shape[0], a.heads, a.vdim)[:, :, t.vdim:] = 0
        for L in self.layers:
            if L.ff != L.ff_p:
                L.gate_up[L.ff:L.ff_p] = 0
                L.gate_up[L.ff_p + L.ff:] = 0
                L.down[:, L.ff:] = 0
        self.lm_head[self.cfg.vocab_size:] = 0
        for L in self.layers:
            if L.type == "mamba2":
                L.in_proj[L.spec.proj_out:] = 0
        return self

    @torch.no_grad()
    def load_state_dict_native(self, sd: dict):
        """Tensors named as in the checkpoint format (module docstring)."""
        def put(p, *names):
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            if tuple(t.shape) != tuple(p.shape):
                raise ValueError(f"{names}: checkpoint shape {tuple(t.shape)} != model {tuple(p.shape)}")
            p.copy_(t.to(p.dtype))

        put(self.embed, "embed")
        put(self.pos, "pos")
        put(self.final_norm, "final.norm")
        if tuple(sd["head"].shape) != (self.cfg.vocab_size, self.cfg.hidden):
            raise ValueError(f"head: checkpoint shape {tuple(sd['head'].shape)}")
        self.lm_head.zero_()
        self.lm_head[:self.cfg.vocab_size].copy_(sd["head"].to(self.lm_head.dtype))
        for i, L in enumerate(self.layers):
            b = f"l{i}."
            put(L.norm1, b + "norm1")
            m = b + "mix."
            if L.type == "attention":
                a, t = L.spec, L.true
                parts = [(m + "q", a.heads, t.dim, a.dim), (m + "k", a.kv_heads, t.dim, a.dim), (m + "v", a.kv_heads, t.vdim, a.vdim)]
                padded = dict(sd)
                for n, h, d, dp in parts:  # [h * d, W] -> [h * dp, W], zero rows behind every head
                    for key, tail in ((n, (sd[n].shape[1],)), (n + ".b", ())):
                        if tuple(sd[key].shape) != (h * d, *tail):
                            raise ValueError(f"{key}: checkpoint shape {tuple(sd[key].shape)} != {(h * d, *tail)}")
                        z = torch.zeros(h, dp, *tail, dtype=sd[key].dtype)
                        z[:, :d] = sd[key].view(h, d, *tail)
                        padded[key] = z.view(h * dp, *tail)
                if tuple(sd[m + "o"].shape) != (L.o.shape[0], a.heads * t.vdim):
                    raise ValueError(f"{m}o: checkpoint shape {tuple(sd[m + 'o'].shape)}")
                z = torch.zeros(L.o.shape[0], a.heads, a.vdim, dtype=sd[m + "o"].dtype)
                z[:, :, :t.vdim] = sd[m + "o"].view(L.o.shape[0], a.heads, t.vdim)
                padded[m + "o"] = z.view(L.o.shape[0], a.heads * a.vdim)
                sd, keep = padded, sd
                put(L.qkv, m + "q", m + "k", m + "v")
                put(L.qkv_b, m + "q.b", m + "k.b", m + "v.b")
                put(L.o, m + "o")
                sd = keep
                put(L.o_b, m + "o.b")
                put(L.r1, m + "r1")
                put(L.r2, m + "r2")
                put(L.pb, m + "pb")
            else:
                if tuple(sd[m + "in"].shape) != (L.spec.proj_out, L.in_proj.shape[1]):
                    raise ValueError(f"{m}in: checkpoint shape {tuple(sd[m + 'in'].shape)}")
                L.in_proj.zero_()
                L.in_proj[:L.spec.proj_out].copy_(sd[m + "in"].to(L.in_proj.dtype))
                put(L.conv_w, m + "conv")
                put(L.conv_b, m + "conv.b")
                put(L.dt_bias, m + "dt_bias")
                put(L.A_log, m + "A_log")
                put(L.D, m + "D")
                put(L.mix_norm, m + "norm")
                put(L.o, m + "o")
            if L.ff:
                g, u, dn = sd[b + "mlp.gate"], sd[b + "mlp.up"], sd[b + "mlp.down"]
                if tuple(g.shape) != (L.ff, L.down.shape[0]) or g.shape != u.shape or tuple(dn.shape) != (L.down.shape[0], L.ff):
                    raise ValueError(f"{b}mlp: checkpoint shapes {tuple(g.shape)}, {tuple(u.shape)}, {tuple(dn.shape)}")
                L.gate_up.zero_()
                L.down.zero_()
                L.gate_up[:L.ff].copy_(g.to(L.gate_up.dtype))
                L.gate_up[L.ff_p:L.ff_p + L.ff].copy_(u.to(L.gate_up.dtype))
                L.down[:, :L.ff].copy_(dn.to(L.down.dtype))
        return self

    def native_state_dict(self) -> dict:
        """The inverse of :meth:`load_state_dict_native` (tests, export)."""
        sd = {"embed": self.embed, "pos": self.pos, "final.norm": self.final_norm,
              "head": self.lm_head[:self.cfg.vocab_size]}
        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            sd[b + "norm1"] = L.norm1
            if L.type == "attention":
                a, t = L.spec, L.true
                nq, nk = a.heads * a.dim, a.kv_heads * a.dim
                for n, w, bb, h, d, dp in (("q", L.qkv[:nq], L.qkv_b[:nq], a.heads, t.dim, a.dim),
                                           ("k", L.qkv[nq:nq + nk], L.qkv_b[nq:nq + nk], a.kv_heads, t.dim, a.dim),
                                           ("v", L.qkv[nq + nk:], L.qkv_b[nq + nk:], a.kv_heads, t.vdim, a.vdim)):
                    sd[m + n] = w.view(h, dp, -1)[:, :d].reshape(h * d, -1)
                    sd[m + n + ".b"] = bb.view(h, dp)[:, :d].reshape(h * d)
                sd[m + "o"] = L.o.view(L.o.shape[0], a.heads, a.vdim)[:, :, :t.vdim].reshape(L.o.shape[0], -1)
                sd.update({m + "o.b": L.o_b, m + "r1": L.r1, m + "r2": L.r2, m + "pb": L.pb})
            else:
                sd.update({m + "in": L.in_proj[:L.spec.proj_out], m + "conv": L.conv_w, m + "conv.b": L.conv_b, m + "dt_bias": L.dt_bias,
                           m + "A_log": L.A_log, m + "D": L.D, m + "norm": L.mix_norm, m + "o": L.o})
            if L.ff:
                sd[b + "mlp.gate"], sd[b + "mlp.up"] = L.gate_up[:L.ff], L.gate_up[L.ff_p:L.ff_p + L.ff]
                sd[b + "mlp.down"] = L.down[:, :L.ff]
        return {k: v.detach().clone().contiguous() for k, v in sd.items()}

    def decode_gemm_shapes(self):
        """(weight, swiglu) of the bias-free projections a decode step runs, one per distinct shape, for
        the engine's decode GEMM routing (ops.tune_decode)."""
        if self.dtype != torch.bfloat16:
            return []   # f32 activations run on the vendor library: nothing to route
        seen, out = set(), []
        for L in self.layers:
            ws = [(L.in_proj, False), (L.o, False)] if L.type == "mamba2" else [(L.qkv, False), (L.o, False)]
            ws += [(L.gate_up, True), (L.down, False)] if L.ff else []
            for w, sw in ws:
                if (tuple(w.shape), sw) not in seen:
                    seen.add((tuple(w.shape), sw))
                    out.append((w, sw))
        # (weights too small to matter are left to the static rule: the tuner streams each from cold HBM copies)
        return [(w, sw) for w, sw in out + [(self.lm_head, False)] if w.numel() >= 1 << 20]

    # ------------------------------------------------------------------ caches
    def make_caches(self, num_blocks: int, block_size: int, num_slots: int) -> list:
        """One entry per layer run: (K cache, V cache) for an attention layer, (conv state, SSM
        state) for a Mamba-2 layer.  Zero-filled: a masked key or a padding row may be read (and
        multiplied by zero), never a NaN pattern left by the allocator."""
        caches = []
        for li, _ in self.runs:
            L = self.layers[li]
            if L.type == "attention":
                if not ops.sigattn_supported(L.spec.heads, L.spec.kv_heads, L.spec.dim, L.spec.vdim, block_size, self.dtype):
                    raise ValueError(f"sigmoid attention kernels do not cover {L.spec} with block size {block_size}")
                ks, vs = L.spec.cache_shapes(num_blocks, block_size)
                caches.append((torch.zeros(ks, dtype=self.dtype, device=self.device),
                               torch.zeros(vs, dtype=self.dtype, device=self.device)))
            else:
                caches.append(L.spec.make_state(num_slots, self.dtype, self.device))
        return caches

    def cache_block_bytes(self, block_size: int) -> int:
        return sum(self.layers[li].spec.bytes_per_token(self.dtype) for li, _ in self.runs
                   if self.layers[li].type == "attention") * block_size

    def state_slot_bytes(self) -> int:
        return sum(self.layers[li].spec.state_bytes(self.dtype) for li, _ in self.runs
                   if self.layers[li].type == "mamba2")

    def kv_bytes_per_token(self) -> int:
        return self.cache_block_bytes(1)

    # ------------------------------------------------------------------ forward
    def _mixer(self, L: LebepelLayer, h, meta: AttnMeta, cache):
        """-> (mixer output without its output bias, that bias or None)."""
        if L.type == "attention":
            # the output projection runs bias-free (decode-sized steps then take the weight-streaming GEMMs):
            # its bias is added by the stream update in f32; the q|k|v bias: see FUSE_QKV_BIAS
            fuse = FUSE_QKV_BIAS
            qkv = ops.linear(h, L.qkv) if fuse else ops.linear(h, L.qkv, L.qkv_b)
            att = sigmoid_paged_attention(qkv, cache[0], cache[1], meta, L.spec, L.r1, L.r2, L.pb, self.cfg.norm_eps,
                                          qkv_bias=L.qkv_b if fuse else None)
            return ops.linear(att, L.o), L.o_b
        return mamba2_mixer(h, L.in_proj, L.conv_w, L.conv_b, L.dt_bias, L.A_log, L.D, L.mix_norm, L.o, L.spec,
                            self.cfg.norm_eps, cache, meta), None

    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches, taps: list = None) -> torch.Tensor:
        """-> normed hidden rows [R, W] that feed the LM head (``meta.logits_idx``, or every row).
        ``taps``: a list that receives a copy of the f32 stream after every layer run (debugging
        and tests; costs one extra pass per layer)."""
        cfg = self.cfg
        m, eps = cfg.residual_mult, cfg.norm_eps
        x, emb = ops.embed_pos(ids, meta.positions, self.embed, self.pos, keep_copy=self.reinject)
        a = b = ab = None
        for run, (li, add_emb) in enumerate(self.runs):
            L = self.layers[li]
            h = ops.stream_rmsnorm(x, a, b, emb if add_emb else None, m, L.norm1, 1.0, eps, out_dtype=self.dtype,
                                   a_bias=ab)
            if taps is not None and run:  # the stream after the previous run, before this pass's re-injection
                taps.append(x - emb if add_emb else x.clone())
            a, ab = self._mixer(L, h, meta, caches[run])
            b = ops.linear(ops.linear_swiglu_any(h, L.gate_up), L.down) if L.ff else None
        if taps is not None:
            d = a.float() if b is None else a.float() + b.float()
            taps.append(x + m * (d if ab is None else d + ab))
        return ops.stream_rmsnorm(x, a, b, None, m, self.final_norm, 1.0, eps, idx=meta.logits_idx, out_dtype=self.dtype,
                                  a_bias=ab)

    def head(self, hidden):
        return ops.linear(hidden, self.lm_head)[:, : self.cfg.vocab_size]

    def logits(self, hidden, gather: bool = True, dtype=torch.float32):
        return ops.softcap(ops.linear(hidden, self.lm_head), self.cfg.logit_softcap)[:, : self.cfg.vocab_size]

    def greedy(self, hidden):
        # the cap is monotonic: the argmax of the raw head output is the argmax of the logits
        return self.tp.greedy_ids(self.head(hidden), self.vocab_lo)


def load_checkpoint_dir(path: str, device="cpu", dtype=torch.bfloat16, name: str = None) -> LebepelModel:
    """Build the model ``path/config.json`` describes and load ``path/*.safetensors`` into it."""
    import json
    from pathlib import Path

    from safetensors.torch import load_file

    d = json.loads((Path(path) / "config.json").read_text())
    cfg = LebepelConfig.from_json(d, name or Path(path).name)
    model = LebepelModel(cfg, SINGLE, dtype, device)
    sd = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        sd.update(load_file(str(f)))
    if not sd:
        raise FileNotFoundError(f"no *.safetensors in {path}")
    return model.load_state_dict_native(sd).eval()
