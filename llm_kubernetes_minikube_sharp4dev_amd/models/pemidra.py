"""Pemidra: a post-norm decoder of linear-state mixers and chunk-masked attention.

    x = embed[token]                                              (f32 stream)
    per layer:  x <- LN1(alpha x + ls1 * mixer(x));  x <- LN2(alpha x + ls2 * ff(x))   (ff may be absent)
    logits = head(LN_final(x))

The sublayers read the normed stream itself.  Mixers, in any order (``cfg.layers``):

* ``retention``      -- ``models.linear_state.retention_mixer``: decayed linear attention;
* ``general_delta``  -- ``models.linear_state.general_delta_mixer``: generalized delta rule;
* ``parallel``       -- ``models.attention.sink_paged_attention`` (softmax with a sink inside fixed chunks of
  positions, paged K/V) beside ``models.linear_state.gated_delta_mixer``, both reading the same input; each
  result RMS-normed over the width with its own weight, half their sum.

Feed-forward: ``W_down (gelu_tanh(W_gate h) * W_up h)``.

MI355X layout decisions:
  * the stream is f32 and each sublayer costs one pass over it: scaled sum, layer scale, layer norm and the
    activation-dtype copy for the next projections are one kernel (``ops.stream_layernorm``); the final norm
    runs only on the rows that feed the LM head;
  * every mixer's input projections are one GEMM (``linear_state.FusedRows``: 16-byte aligned column blocks);
  * all three recurrences run on one scan kernel over slot-indexed f32 states (``ops.delta_scan``), so
    portions of prompts, decode rows and mixed batches are one code path; decays, gates, unit norms and
    softmax statistics are f32 inside the kernels.

Checkpoint format: ``config.json`` (``PemidraConfig.from_json``) and ``model.safetensors`` with ``embed``,
``l<i>.norm1`` (+ ``.b``), ``l<i>.ls1``, ``l<i>.mix.*``, ``l<i>.norm2``, ``l<i>.ls2``, ``l<i>.mlp.*``, ``final.norm``
(+ ``.b``), ``head``; linear weights [out, in].  The ranks of the two-layer projections are read from the
tensors' shapes (``ranks_from_state_dict``).
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops
from ..parallel.tp import SINGLE, TPGroup
from .attention import AttnMeta, SinkAttnSpec, sink_paged_attention
from .configs import PemidraConfig, pad_vocab
from .linear_state import (FusedRows, GatedDeltaSpec, GeneralDeltaSpec, RetentionSpec, fused_mult, gated_delta_mixer,
                           general_delta_mixer, retention_mixer)


def _p(*shape, **kw):
    return nn.Parameter(torch.zeros(*shape, **kw), requires_grad=False)


def _pad8(n: int) -> int:
    return -(-int(n) // 8) * 8


class _Retention(nn.Module):
    """Weights of a retention mixer under checkpoint prefix ``mix.``."""

    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        s = self.spec = RetentionSpec.from_dict(m)
        self.rows = s.rows(W)
        self.w_in = _p(self.rows.total, W, **e)
        self.decay = _p(s.heads, **f)
        self.o = _p(W, s.heads * s.vdim, **e)
        self.segments = {"q": "q", "k": "k", "v": "v", "g": "g"}

    def init_constants(self):
        self.decay.copy_(torch.tensor(self.spec.decay, dtype=torch.float32))


class _GeneralDelta(nn.Module):
    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        s = self.spec = GeneralDeltaSpec.from_dict(m)
        self.rows = s.rows(W)
        self.w_in = _p(self.rows.total, W, **e)
        self.w2 = _p(s.inner, _pad8(s.lora), **e)     # zero columns behind the rank
        self.w0, self.a_b, self.norm = _p(s.inner, **f), _p(s.inner, **f), _p(s.inner, **f)
        self.o = _p(W, s.inner, **e)
        self.segments = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "w1": "w1"}


class _GatedDelta(nn.Module):
    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        s = self.spec = GatedDeltaSpec.from_dict(m)
        self.rows = s.rows(W)
        self.w_in = _p(self.rows.total, W, **e)
        self.conv_w = _p(s.conv_channels(), s.conv, **f)          # zero rows at the alignment padding
        self.a2 = _p(s.heads * s.dim, _pad8(s.lora_a), **e)
        self.g2 = _p(s.heads * s.vdim, _pad8(s.lora_g), **e)
        self.dt_bias, self.A_log = _p(s.heads * s.dim, **f), _p(s.heads, **f)
        self.norm = _p(s.heads * s.vdim, **f)                     # the per-head weight, repeated for every head
        self.o = _p(W, s.heads * s.vdim, **e)
        self.segments = {"q": "q", "k": "k", "v": "v", "b": "b", "a1": "a1", "g1": "g1"}


class _SinkAttention(nn.Module):
    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        t = self.true = SinkAttnSpec.from_dict(m)                 # the checkpoint's sizes
        # head sizes padded to the kernels' 8-element fragments with zero weight rows / columns; the norms'
        # divisors stay the true sizes
        s = self.spec = SinkAttnSpec(t.heads, t.kv_heads, _pad8(t.dim), _pad8(t.vdim), t.scale, t.mask_kind, t.mask_size,
                                     t.rot_dims, t.rot_base, t.sink, t.v_unit)
        self.rows = FusedRows([("q", s.heads * s.dim), ("k", s.kv_heads * s.dim), ("v", s.kv_heads * s.vdim), ("g", s.heads)],
                              fused_mult(W))
        self.w_in = _p(self.rows.total, W, **e)
        self.q_norm, self.k_norm = _p(s.dim, **f), _p(s.dim, **f)
        self.temp, self.hscale = _p(s.heads, **f), _p(s.heads, **f)     # hscale = scale * temp, what the kernels read
        self.inv_freq = _p(max(s.rot_dims // 2, 1), **f)
        self.o = _p(W, s.heads * s.vdim, **e)

    def init_constants(self):
        if self.spec.rot_dims:
            self.inv_freq.copy_(self.spec.inv_freq(self.inv_freq.device))
        self.hscale.copy_(self.temp * self.spec.scale)


class PemidraLayer(nn.Module):
    def __init__(self, cfg: PemidraConfig, spec, dtype, device):
        super().__init__()
        W = cfg.hidden
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)   # norms, scales and per-channel constants stay f32
        self.type = spec.type
        self.norm1, self.norm1_b, self.ls1 = _p(W, **f), _p(W, **f), _p(W, **f)
        if spec.type == "retention":
            self.mix = _Retention(spec.mixer, W, e, f)
        elif spec.type == "general_delta":
            self.mix = _GeneralDelta(spec.mixer, W, e, f)
        else:
            self.left = _SinkAttention(spec.mixer["left"], W, e, f)
            self.right = _GatedDelta(spec.mixer["right"], W, e, f)
            self.left_out, self.right_out = _p(W, **f), _p(W, **f)
        self.ff = int(spec.mlp["ff"]) if spec.mlp else 0
        self.ff_p = _pad8(self.ff)     # padded with zero gate / up rows and down columns (16-byte rows)
        if self.ff:
            self.gate_up, self.down = _p(2 * self.ff_p, W, **e), _p(W, self.ff_p, **e)
            self.norm2, self.norm2_b, self.ls2 = _p(W, **f), _p(W, **f), _p(W, **f)

    def state_specs(self):
        return [self.mix.spec] if self.type != "parallel" else [self.right.spec]


def ranks_from_state_dict(cfg: PemidraConfig, sd: dict) -> PemidraConfig:
    """The ranks of the two-layer projections are sizes that only the tensors' shapes give: note them in
    the mixers' dicts before the model is built."""
    for i, l in enumerate(cfg.layers):
        m = f"l{i}.mix."
        if l.type == "general_delta":
            l.mixer["lora"] = int(sd[m + "w1"].shape[0])
        elif l.type == "parallel":
            l.mixer["right"]["lora_a"] = int(sd[m + "right.a1"].shape[0])
            l.mixer["right"]["lora_g"] = int(sd[m + "right.g1"].shape[0])
    return cfg


class PemidraModel(nn.Module):
    stateful = True            # recurrent state per sequence: no prefix reuse, no multi-row decode of one sequence

    def __init__(self, cfg: PemidraConfig, tp: TPGroup = SINGLE, dtype=torch.bfloat16, device="cpu"):
        super().__init__()
        if tp.enabled:
            raise NotImplementedError("the Pemidra decoder runs on one GPU (no tensor-parallel sharding)")
        self.cfg, self.tp, self.dtype, self.device = cfg, tp, dtype, torch.device(device)
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)
        self.vocab_lo, self.vocab_local = 0, cfg.vocab_size
        self.embed = _p(cfg.vocab_size, cfg.hidden, **e)
        self.layers = nn.ModuleList([PemidraLayer(cfg, l, dtype, device) for l in cfg.layers])
        self.final_norm, self.final_norm_b = _p(cfg.hidden, **f), _p(cfg.hidden, **f)
        # head rows padded (zero rows) so that logits rows start 32-byte aligned for the sampling kernels
        self.lm_head = _p(pad_vocab(cfg.vocab_size, 64), cfg.hidden, **e)
        att = [l.left.spec for l in self.layers if l.type == "parallel"]
        self.hq = max((a.heads for a in att), default=1)
        self.hkv = max((a.kv_heads for a in att), default=1)
        self.D = max((max(a.dim, a.vdim) for a in att), default=16)

    # ------------------------------------------------------------------ weights
    def _finish(self):
        for L in self.layers:
            for m in ((L.mix,) if L.type != "parallel" else (L.left, L.right)):
                if hasattr(m, "init_constants"):
                    m.init_constants()
        return self

    @torch.no_grad()
    def random_init(self, seed: int = 0):
        """Random weights of a scale that keeps every mechanism active (decays away from 0 and 1, scores of
        order one), written through the checkpoint names so that padding stays zero."""
        return self.load_state_dict_native(random_state_dict(self.cfg, seed))

    @torch.no_grad()
    def load_state_dict_native(self, sd: dict):
        """Tensors named as in the checkpoint format (module docstring)."""
        cfg, W = self.cfg, self.cfg.hidden

        def get(name, *shape):
            t = sd[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(t.shape)} != {tuple(shape)}")
            return t

        def put(p, name):
            p.copy_(get(name, *p.shape).to(p.dtype))

        def fuse(mod, prefix, sizes: dict):
            """Fill the fused input projection from its segments' tensors (padding rows stay zero)."""
            mod.w_in.zero_()
            for seg, rows in sizes.items():
                o = mod.rows.off[seg]
                mod.w_in[o:o + rows].copy_(get(prefix + seg, rows, W).to(mod.w_in.dtype))

        put(self.embed, "embed")
        put(self.final_norm, "final.norm")
        put(self.final_norm_b, "final.norm.b")
        self.lm_head.zero_()
        self.lm_head[:cfg.vocab_size].copy_(get("head", cfg.vocab_size, W).to(self.lm_head.dtype))
        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            put(L.norm1, b + "norm1")
            put(L.norm1_b, b + "norm1.b")
            put(L.ls1, b + "ls1")
            if L.type == "retention":
                s = L.mix.spec
                fuse(L.mix, m, {"q": s.heads * s.dim, "k": s.heads * s.dim, "v": s.heads * s.vdim, "g": s.heads * s.vdim})
                put(L.mix.o, m + "o")
            elif L.type == "general_delta":
                s = L.mix.spec
                n = s.inner
                fuse(L.mix, m, {"r": n, "k": n, "v": n, "g": n, "a": n, "w1": s.lora})
                L.mix.w2.zero_()
                L.mix.w2[:, :s.lora].copy_(get(m + "w2", n, s.lora).to(L.mix.w2.dtype))
                put(L.mix.w0, m + "w0")
                put(L.mix.a_b, m + "a.b")
                put(L.mix.norm, m + "norm")
                put(L.mix.o, m + "o")
            else:
                self._load_left(L.left, m + "left.", get, put)
                self._load_right(L.right, m + "right.", get, put, fuse)
                put(L.left_out, m + "left.out")
                put(L.right_out, m + "right.out")
            if L.ff:
                g, u, dn = get(b + "mlp.gate", L.ff, W), get(b + "mlp.up", L.ff, W), get(b + "mlp.down", W, L.ff)
                L.gate_up.zero_()
                L.down.zero_()
                L.gate_up[:L.ff].copy_(g.to(L.gate_up.dtype))
                L.gate_up[L.ff_p:L.ff_p + L.ff].copy_(u.to(L.gate_up.dtype))
                L.down[:, :L.ff].copy_(dn.to(L.down.dtype))
                put(L.norm2, b + "norm2")
                put(L.norm2_b, b + "norm2.b")
                put(L.ls2, b + "ls2")
        return self._finish()

    def _load_left(self, A, m, get, put):
        a, t, W = A.spec, A.true, self.cfg.hidden
        A.w_in.zero_()
        for seg, h, d, dp in (("q", a.heads, t.dim, a.dim), ("k", a.kv_heads, t.dim, a.dim), ("v", a.kv_heads, t.vdim, a.vdim)):
            o = A.rows.off[seg]
            A.w_in[o:o + h * dp].view(h, dp, W)[:, :d].copy_(get(m + seg, h * d, W).view(h, d, W).to(A.w_in.dtype))
        o = A.rows.off["g"]
        A.w_in[o:o + a.heads].copy_(get(m + "g", a.heads, W).to(A.w_in.dtype))
        for p, n in ((A.q_norm, "q.norm"), (A.k_norm, "k.norm")):
            p.zero_()
            p[:t.dim].copy_(get(m + n, t.dim).to(p.dtype))
        put(A.temp, m + "temp")
        A.o.zero_()
        A.o.view(W, a.heads, a.vdim)[:, :, :t.vdim].copy_(get(m + "o", W, a.heads * t.vdim).view(W, a.heads, t.vdim).to(A.o.dtype))

    def _load_right(self, R, m, get, put, fuse):
        s = R.spec
        nk, nv = s.kv_heads * s.dim, s.heads * s.vdim
        fuse(R, m, {"q": nk, "k": nk, "v": nv, "b": s.heads, "a1": s.lora_a, "g1": s.lora_g})
        R.conv_w.zero_()
        for seg, n in (("q", nk), ("k", nk), ("v", nv)):
            o = R.rows.off[seg]
            R.conv_w[o:o + n].copy_(get(m + seg + ".conv", n, s.conv).to(R.conv_w.dtype))
        R.a2.zero_()
        R.a2[:, :s.lora_a].copy_(get(m + "a2", s.heads * s.dim, s.lora_a).to(R.a2.dtype))
        R.g2.zero_()
        R.g2[:, :s.lora_g].copy_(get(m + "g2", nv, s.lora_g).to(R.g2.dtype))
        put(R.dt_bias, m + "dt_bias")
        put(R.A_log, m + "A_log")
        R.norm.copy_(get(m + "norm", s.vdim).to(R.norm.dtype).repeat(s.heads))
        put(R.o, m + "o")

    def native_state_dict(self) -> dict:
        """The inverse of :meth:`load_state_dict_native` (tests, export)."""
        cfg, W = self.cfg, self.cfg.hidden
        sd = {"embed": self.embed, "final.norm": self.final_norm, "final.norm.b": self.final_norm_b,
              "head": self.lm_head[:cfg.vocab_size]}

        def unfuse(mod, prefix, sizes):
            for seg, rows in sizes.items():
                o = mod.rows.off[seg]
                sd[prefix + seg] = mod.w_in[o:o + rows]

        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            sd.update({b + "norm1": L.norm1, b + "norm1.b": L.norm1_b, b + "ls1": L.ls1})
            if L.type == "retention":
                s = L.mix.spec
                unfuse(L.mix, m, {"q": s.heads * s.dim, "k": s.heads * s.dim, "v": s.heads * s.vdim, "g": s.heads * s.vdim})
                sd[m + "o"] = L.mix.o
            elif L.type == "general_delta":
                s = L.mix.spec
                n = s.inner
                unfuse(L.mix, m, {"r": n, "k": n, "v": n, "g": n, "a": n, "w1": s.lora})
                sd.update({m + "w2": L.mix.w2[:, :s.lora], m + "w0": L.mix.w0, m + "a.b": L.mix.a_b, m + "norm": L.mix.norm,
                           m + "o": L.mix.o})
            else:
                A, R = L.left, L.right
                a, t = A.spec, A.true
                for seg, h, d, dp in (("q", a.heads, t.dim, a.dim), ("k", a.kv_heads, t.dim, a.dim),
                                      ("v", a.kv_heads, t.vdim, a.vdim)):
                    o = A.rows.off[seg]
                    sd[m + "left." + seg] = A.w_in[o:o + h * dp].view(h, dp, W)[:, :d].reshape(h * d, W)
                o = A.rows.off["g"]
                sd.update({m + "left.g": A.w_in[o:o + a.heads], m + "left.q.norm": A.q_norm[:t.dim], m + "left.k.norm": A.k_norm[:t.dim],
                           m + "left.temp": A.temp, m + "left.out": L.left_out, m + "right.out": L.right_out,
                           m + "left.o": A.o.view(W, a.heads, a.vdim)[:, :, :t.vdim].reshape(W, -1)})
                s = R.spec
                nk, nv = s.kv_heads * s.dim, s.heads * s.vdim
                unfuse(R, m + "right.", {"q": nk, "k": nk, "v": nv, "b": s.heads, "a1": s.lora_a, "g1": s.lora_g})
                for seg, n in (("q", nk), ("k", nk), ("v", nv)):
                    o = R.rows.off[seg]
                    sd[m + f"right.{seg}.conv"] = R.conv_w[o:o + n]
                sd.update({m + "right.a2": R.a2[:, :s.lora_a], m + "right.g2": R.g2[:, :s.lora_g], m + "right.dt_bias": R.dt_bias,
                           m + "right.A_log": R.A_log, m + "right.norm": R.norm[:s.vdim], m + "right.o": R.o})
            if L.ff:
                sd.update({b + "mlp.gate": L.gate_up[:L.ff], b + "mlp.up": L.gate_up[L.ff_p:L.ff_p + L.ff], b + "mlp.down": L.down[:, :L.ff],
                           b + "norm2": L.norm2, b + "norm2.b": L.norm2_b, b + "ls2": L.ls2})
        return {k: v.detach().clone().contiguous() for k, v in sd.items()}

    def decode_gemm_shapes(self):
        """(weight, swiglu) of the projections a decode step runs, one per distinct shape, for the engine's
        decode GEMM routing (ops.tune_decode)."""
        if self.dtype != torch.bfloat16:
            return []   # f32 activations run on the vendor library: nothing to route
        seen, out = set(), []
        for L in self.layers:
            mods = (L.mix,) if L.type != "parallel" else (L.left, L.right)
            ws = [w for m in mods for w in (m.w_in, m.o)] + ([L.gate_up, L.down] if L.ff else [])
            for w in ws:
                if tuple(w.shape) not in seen:
                    seen.add(tuple(w.shape))
                    out.append((w, False))
        return [(w, sw) for w, sw in out + [(self.lm_head, False)] if w.numel() >= 1 << 20]

    # ------------------------------------------------------------------ caches
    def make_caches(self, num_blocks: int, block_size: int, num_slots: int) -> list:
        """One entry per layer: the mixer's f32 state (plus, for a parallel layer, the paged K / V caches
        in front and the convolution state).  Zero-filled: a masked key or a padding row may be read (and
        multiplied by zero), never a NaN pattern left by the allocator."""
        caches = []
        for L in self.layers:
            if L.type == "parallel":
                a = L.left.spec
                if not ops.sigattn_supported(a.heads, a.kv_heads, a.dim, a.vdim, block_size, self.dtype):
                    raise ValueError(f"attention kernels do not cover {a} with block size {block_size}")
                ks, vs = a.cache_shapes(num_blocks, block_size)
                kv = (torch.zeros(ks, dtype=self.dtype, device=self.device), torch.zeros(vs, dtype=self.dtype, device=self.device))
                caches.append(kv + L.right.spec.make_state(num_slots, self.dtype, self.device))
            else:
                caches.append(L.mix.spec.make_state(num_slots, self.dtype, self.device))
        return caches

    def cache_block_bytes(self, block_size: int) -> int:
        return sum(L.left.spec.bytes_per_token(self.dtype) for L in self.layers if L.type == "parallel") * block_size

    def state_slot_bytes(self) -> int:
        return sum(s.state_bytes(self.dtype) for L in self.layers for s in L.state_specs())

    def kv_bytes_per_token(self) -> int:
        return self.cache_block_bytes(1)

    # ------------------------------------------------------------------ forward
    def _mixer(self, L: PemidraLayer, h, meta: AttnMeta, cache):
        eps = self.cfg.norm_eps
        if L.type == "retention":
            M = L.mix
            return retention_mixer(h, M.w_in, M.rows, M.decay, M.o, M.spec, eps, cache, meta, self.dtype)
        if L.type == "general_delta":
            M = L.mix
            return general_delta_mixer(h, M.w_in, M.rows, M.w2, M.w0, M.a_b, M.norm, M.o, M.spec, eps, cache, meta, self.dtype)
        A, R = L.left, L.right
        u = ops.linear(h, A.w_in)
        att = sink_paged_attention(u, cache[0], cache[1], meta, A.spec, A.q_norm, A.k_norm, A.inv_freq, A.hscale, eps,
                                   gate_col=A.rows.off["g"], norm_dim=A.true.dim, norm_vdim=A.true.vdim)
        left = ops.linear(att, A.o)
        right = gated_delta_mixer(h, R.w_in, R.rows, R.conv_w, R.a2, R.dt_bias, R.A_log, R.g2, R.norm, R.o, R.spec, eps,
                                  cache[2:], meta, self.dtype)
        return ops.dual_rmsnorm_mean(left, L.left_out, right, L.right_out, eps)

    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches, taps: list = None) -> torch.Tensor:
        """-> normed hidden rows [R, W] that feed the LM head (``meta.logits_idx``, or every row).
        ``taps``: a list that receives a copy of the f32 stream after every layer (debugging and tests)."""
        cfg = self.cfg
        alpha, eps = cfg.postln_alpha, cfg.norm_eps
        x, h = ops.embed_stream(ids, self.embed, self.dtype)
        for i, L in enumerate(self.layers):
            y = self._mixer(L, h, meta, caches[i])
            h = ops.stream_layernorm(x, y, L.ls1, alpha, L.norm1, L.norm1_b, eps, self.dtype)
            if L.ff:
                y = ops.linear(ops.gelu_tanh_mul(ops.linear(h, L.gate_up)), L.down)
                h = ops.stream_layernorm(x, y, L.ls2, alpha, L.norm2, L.norm2_b, eps, self.dtype)
            if taps is not None:
                taps.append(x.clone())
        idx = meta.logits_idx
        if idx is None:
            idx = torch.arange(x.shape[0], dtype=torch.long, device=x.device)
        return ops.stream_layernorm(x, None, None, 1.0, self.final_norm, self.final_norm_b, eps, self.dtype, idx=idx)

    def head(self, hidden):
        return ops.linear(hidden, self.lm_head)[:, : self.cfg.vocab_size]

    def logits(self, hidden, gather: bool = True, dtype=torch.float32):
        lg = self.head(hidden)
        return lg if dtype is None else lg.to(dtype)

    def greedy(self, hidden):
        return self.tp.greedy_ids(self.head(hidden), self.vocab_lo)


def random_state_dict(cfg: PemidraConfig, seed: int = 0) -> dict:
    """Random f32 tensors under the checkpoint names for ``cfg`` (presets, benchmarks, tests)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden

    def rn(*shape, scale=1.0, shift=0.0):
        return torch.randn(*shape, generator=g) * scale + shift

    def lin(out, inp, gain=1.0):
        return rn(out, inp, scale=gain / math.sqrt(inp))

    sd = {"embed": rn(cfg.vocab_size, W), "final.norm": rn(W, scale=0.1, shift=1.0), "final.norm.b": rn(W, scale=0.1),
          "head": lin(cfg.vocab_size, W)}
    for i, l in enumerate(cfg.layers):
        b, m = f"l{i}.", f"l{i}.mix."
        sd.update({b + "norm1": rn(W, scale=0.1, shift=1.0), b + "norm1.b": rn(W, scale=0.1), b + "ls1": rn(W, scale=0.2, shift=1.0)})
        if l.type == "retention":
            s = RetentionSpec.from_dict(l.mixer)
            sd.update({m + "q": lin(s.heads * s.dim, W), m + "k": lin(s.heads * s.dim, W), m + "v": lin(s.heads * s.vdim, W),
                       m + "g": lin(s.heads * s.vdim, W), m + "o": lin(W, s.heads * s.vdim)})
        elif l.type == "general_delta":
            s = GeneralDeltaSpec.from_dict(l.mixer)
            n = s.inner
            sd.update({m + k: lin(n, W) for k in ("r", "k", "v", "g", "a")})
            sd.update({m + "w1": lin(s.lora, W), m + "w2": lin(n, s.lora, 2.0), m + "w0": rn(n), m + "a.b": rn(n, scale=0.5),
                       m + "norm": rn(n, scale=0.1, shift=1.0), m + "o": lin(W, n)})
        else:
            a = SinkAttnSpec.from_dict(l.mixer["left"])
            p = m + "left."
            sd.update({p + "q": lin(a.heads * a.dim, W), p + "k": lin(a.kv_heads * a.dim, W), p + "v": lin(a.kv_heads * a.vdim, W),
                       p + "q.norm": rn(a.dim, scale=0.2, shift=1.0), p + "k.norm": rn(a.dim, scale=0.2, shift=1.0),
                       p + "temp": rn(a.heads, scale=0.3, shift=1.5), p + "g": lin(a.heads, W), p + "o": lin(W, a.heads * a.vdim),
                       p + "out": rn(W, scale=0.1, shift=1.0)})
            s = GatedDeltaSpec.from_dict(l.mixer["right"])
            p = m + "right."
            nk, nv = s.kv_heads * s.dim, s.heads * s.vdim
            sd.update({p + "q": lin(nk, W), p + "k": lin(nk, W), p + "v": lin(nv, W), p + "b": lin(s.heads, W),
                       p + "q.conv": rn(nk, s.conv, scale=0.5), p + "k.conv": rn(nk, s.conv, scale=0.5),
                       p + "v.conv": rn(nv, s.conv, scale=0.5), p + "a1": lin(s.lora_a, W), p + "a2": lin(s.heads * s.dim, s.lora_a),
                       p + "dt_bias": rn(s.heads * s.dim, scale=0.5, shift=-1.0), p + "A_log": rn(s.heads, scale=0.3),
                       p + "g1": lin(s.lora_g, W), p + "g2": lin(nv, s.lora_g), p + "norm": rn(s.vdim, scale=0.1, shift=1.0),
                       p + "o": lin(W, nv), p + "out": rn(W, scale=0.1, shift=1.0)})
        if l.mlp:
            ff = int(l.mlp["ff"])
            sd.update({b + "mlp.gate": lin(ff, W), b + "mlp.up": lin(ff, W), b + "mlp.down": lin(W, ff),
                       b + "norm2": rn(W, scale=0.1, shift=1.0), b + "norm2.b": rn(W, scale=0.1), b + "ls2": rn(W, scale=0.2, shift=1.0)})
    return sd
