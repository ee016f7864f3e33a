"""The Pemidra decoder's mechanisms, each alone, against the plain float64 implementations of
``pemidra_oracle``: the framework's mixers over a paged cache / state slots, whole sequences, cut into
portions and decoded token by token, on the CPU path and (``gpu`` marker) on the HIP kernels in f32 and
bf16.  Where random weights would hide a fault (a chunk's edge, a far key, the sink, a value written long
ago) the inputs are made so that it shows."""
import math

import pytest
import torch

import pemidra_oracle as O
from llm_kubernetes_minikube_sharp4dev_amd import ops
from llm_kubernetes_minikube_sharp4dev_amd.models import PemidraConfig, build_decoder
from llm_kubernetes_minikube_sharp4dev_amd.models.attention import AttnMeta

CPU32 = pytest.param("cpu", torch.float32, id="cpu-f32")
GPU32 = pytest.param("cuda", torch.float32, id="gpu-f32", marks=pytest.mark.gpu)
GPU16 = pytest.param("cuda", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)
ALL = [CPU32, GPU32, GPU16]
BS = 16


def tol(dtype):
    return 3e-5 if dtype == torch.float32 else 4e-2


def rel_err(got, want):
    want = want.double()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9))


def rnd(g, *shape, scale=1.0):
    return torch.randn(*shape, generator=g, dtype=torch.float64) * scale


def q16(t):
    """Values a bf16 tensor holds exactly, so both sides of a comparison start from the same numbers."""
    return t.to(torch.bfloat16).to(torch.float64)


def step_meta(seqs, device):
    """AttnMeta of one step, as the model runner lays it out: ``seqs`` = [(start, n, block table, state
    slot, decode row?)], prompt portions first, then decode rows (n == 1)."""
    pre = [s for s in seqs if not s[4]]
    dec = [s for s in seqs if s[4]]
    pos, slots, cu, ctx_p, ctx_d, st = [], [], [0], [], [], []
    for start, n, table, slot, _ in pre + dec:
        for p in range(start, start + n):
            pos.append(p)
            slots.append(table[p // BS] * BS + p % BS)
        st.append(slot)
    for start, n, *_ in pre:
        cu.append(cu[-1] + n)
        ctx_p.append(start + n)
    i32 = dict(dtype=torch.int32, device=device)

    def tables(group):
        w = max(len(s[2]) for s in group)
        return torch.tensor([list(s[2]) + [0] * (w - len(s[2])) for s in group], **i32)

    m = AttnMeta(positions=torch.tensor(pos, **i32), slots=torch.tensor(slots, **i32), num_prefill_tokens=cu[-1],
                 num_prefill_seqs=len(pre), num_decode=len(dec))
    if pre:
        m.cu_q, m.ctx_lens_p, m.block_tables_p = torch.tensor(cu, **i32), torch.tensor(ctx_p, **i32), tables(pre)
        m.q_lens_cpu, m.ctx_lens_cpu = [s[1] for s in pre], ctx_p
    if dec:
        m.block_tables_d, m.ctx_lens_d = tables(dec), torch.tensor([s[0] + 1 for s in dec], **i32)
    lens = [s[1] for s in pre] + [1] * len(dec)
    m.seq_cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), **i32)
    m.state_slots = torch.tensor(st, **i32)
    m.max_seq_len = max(lens)
    return m


def one_layer(kind, mixer, W, device, dtype, seed=5, eps=1e-5):
    """A one-layer model of the mechanism (random weights through the checkpoint names) and its tensors."""
    cfg = PemidraConfig.from_json({"architecture": "Pemidra", "vocab": 11, "width": W, "norm": {"eps": eps}, "postln_alpha": 1.0,
                                   "layers": [{"type": kind, "mixer": mixer, "mlp": None}]})
    m = build_decoder(cfg, device=device, dtype=dtype, seed=seed)
    sd = {k: v.cpu().double() for k, v in m.native_state_dict().items()}
    return m, sd


def run_mixer(m, h, cuts, device, dtype, slot=1, blocks=None, nblocks=24, caches=None):
    """The layer's mixer over ``h`` [T, W] fed in portions of the sizes ``cuts`` (the rest as decode rows)."""
    T = h.shape[0]
    blocks = blocks or list(range(nblocks - 1, nblocks - 1 - (T + BS - 1) // BS, -1))   # pages in descending order
    caches = caches or m.make_caches(nblocks, BS, 3)
    out, at, sizes = [], 0, list(cuts)
    while at < T:
        dec = not sizes
        n = 1 if dec else min(sizes.pop(0), T - at)
        meta = step_meta([(at, n, blocks, slot, dec)], device)
        with torch.inference_mode():
            y = m._mixer(m.layers[0], h[at:at + n].to(dtype).to(device).contiguous(), meta, caches[0])
        out.append(y.float().cpu())
        at += n
    return torch.cat(out)


RET = {"heads": 3, "dim": 12, "vdim": 20, "decay": [0.9, 0.995, 1.0]}
GEN = {"heads": 2, "dim": 24, "lora": 5}
PAR = {"left": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.3, "mask": {"size": 13},
                "rot": {"dims": 10, "base": 50.0}},
       "right": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 20, "conv": 3, "lora_a": 6, "lora_g": 9}}
KINDS = {"retention": (RET, O.retention), "general_delta": (GEN, O.general_delta), "parallel": (PAR, O.parallel_mixer)}


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("kind", list(KINDS))
def test_mixer_whole_portions_and_token_by_token(kind, device, dtype):
    """A whole prompt in one step, token by token from the first token on, and portions of 1, 2, 2, 3,
    16, 17, 5 tokens followed by decode rows give the oracle's result at every position."""
    mixer, fn = KINDS[kind]
    W, T = 40, 61
    m, sd = one_layer(kind, mixer, W, device, dtype)
    h = q16(rnd(torch.Generator().manual_seed(3), T, W))
    want = fn(h, sd, "l0.mix.", mixer, 1e-5)
    for cuts in ([T], [1], [1, 2, 2, 3, 16, 17, 5], [30, 2, 29]):
        got = run_mixer(m, h, cuts, device, dtype)
        assert rel_err(got, want) < tol(dtype), (cuts, rel_err(got, want))


@pytest.mark.parametrize("device,dtype", ALL)
def test_head_sizes_beyond_one_lane_slice(device, dtype):
    """Key sizes that take the scan's widest row split (more than 128 rows), a value size that is not a
    multiple of a wave's columns, one head, a decay of exactly 1."""
    W, T = 48, 37
    h = q16(rnd(torch.Generator().manual_seed(4), T, W))
    for kind, mixer in (("general_delta", {"heads": 1, "dim": 136, "lora": 3}),
                        ("retention", {"heads": 2, "dim": 72, "vdim": 40, "decay": [1.0, 0.5]})):
        m, sd = one_layer(kind, mixer, W, device, dtype)
        want = KINDS[kind][1](h, sd, "l0.mix.", mixer, 1e-5)
        for cuts in ([T], [9, 2]):
            assert rel_err(run_mixer(m, h, cuts, device, dtype), want) < tol(dtype), (kind, cuts)


@pytest.mark.parametrize("device,dtype", ALL)
def test_retention_keeps_a_value_written_long_ago(device, dtype):
    """Decay 1 keeps the first token's write for good: with keys that do not overlap later ones the read-out
    300 decode steps later returns it; decay 0.5 has lost it."""
    W, T = 16, 301
    mixer = {"heads": 2, "dim": 8, "vdim": 8, "decay": [1.0, 0.5]}
    m, sd = one_layer("retention", mixer, W, device, dtype)
    g = torch.Generator().manual_seed(6)
    h = q16(rnd(g, T, W, scale=0.05))
    h[0], h[-1] = q16(rnd(g, W)), 0.0
    h[-1] = h[0]           # the last query lines up with the first key
    want = O.retention(h, sd, "l0.mix.", mixer, 1e-5)
    got = run_mixer(m, h, [5], device, dtype)
    assert rel_err(got[-1], want[-1]) < tol(dtype)
    assert rel_err(got, want) < tol(dtype)


@pytest.mark.parametrize("device,dtype", ALL)
def test_state_slots_start_from_zero_and_are_independent(device, dtype):
    """Two sequences in one step with different slots, then a new sequence in a slot that holds an old
    state (and a poisoned convolution state): each equals its run alone."""
    kind, (mixer, fn) = "parallel", KINDS["parallel"]
    W = 40
    m, sd = one_layer(kind, mixer, W, device, dtype)
    g = torch.Generator().manual_seed(7)
    ha, hb, hc = q16(rnd(g, 22, W)), q16(rnd(g, 9, W)), q16(rnd(g, 15, W))
    caches = m.make_caches(12, BS, 3)
    for c in caches[0][2:]:
        c.fill_(float("nan") if c.dtype != torch.float32 else 1e30)   # whatever an earlier owner left
    ta, tb = [3, 7], [5]
    with torch.inference_mode():
        meta = step_meta([(0, 20, ta, 2, False), (0, 8, tb, 0, False)], device)
        y1 = m._mixer(m.layers[0], torch.cat([ha[:20], hb[:8]]).to(dtype).to(device), meta, caches[0]).float().cpu()
        meta = step_meta([(20, 2, ta, 2, False), (8, 1, tb, 0, True)], device)
        y2 = m._mixer(m.layers[0], torch.cat([ha[20:], hb[8:]]).to(dtype).to(device), meta, caches[0]).float().cpu()
        # c takes b's slot and pages
        meta = step_meta([(0, 15, tb, 0, False)], device)
        y3 = m._mixer(m.layers[0], hc.to(dtype).to(device), meta, caches[0]).float().cpu()
    for got, hh in ((torch.cat([y1[:20], y2[:2]]), ha), (torch.cat([y1[20:], y2[2:]]), hb), (y3, hc)):
        assert rel_err(got, fn(hh, sd, "l0.mix.", mixer, 1e-5)) < tol(dtype)


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("dk,dv,H,Hk", [(8, 10, 2, 1), (24, 16, 4, 2), (48, 64, 2, 2), (96, 40, 3, 1), (200, 72, 1, 1)])
def test_scan_forms_agree_with_the_recurrence(dk, dv, H, Hk, device, dtype):
    """The scan op alone, both lane splits of the GPU kernel (4 and 16 lanes per state column), with and
    without the removal term, two sequences of unequal length continued from an earlier state, against the
    recurrence written out in float64."""
    g = torch.Generator().manual_seed(dk)
    lens, T = [19, 6], 25
    q, k, v = q16(rnd(g, T, Hk * dk, scale=0.4)), q16(rnd(g, T, Hk * dk, scale=0.4)), q16(rnd(g, T, H * dv))
    w = torch.rand(T, H * dk, generator=g, dtype=torch.float64).float().double() * 0.5 + 0.5
    p, z = rnd(g, T, H * dk, scale=0.3).float().double(), rnd(g, T, H * dk, scale=0.3).float().double()
    wh = torch.tensor([0.9, 1.0, 0.5, 0.75][:H], dtype=torch.float64)
    S0 = rnd(g, 3, H, dk, dv, scale=0.2).float().double()
    i32 = dict(dtype=torch.int32, device=device)
    cu, slots = torch.tensor([0, 19, 25], **i32), torch.tensor([2, 0], **i32)
    pos = torch.tensor(list(range(5, 24)) + list(range(0, 6)), **i32)      # the first continues, the second starts fresh
    for full in (True, False):
        want = torch.zeros(T, H, dv, dtype=torch.float64)
        end = {}
        for s, (r0, n, slot, fresh) in enumerate(((0, 19, 2, False), (19, 6, 0, True))):
            for h in range(H):
                S = torch.zeros(dk, dv, dtype=torch.float64) if fresh else S0[slot, h].clone()
                kh = h // (H // Hk)
                for t in range(r0, r0 + n):
                    kk = k[t, kh * dk:(kh + 1) * dk] * (1.0 if full else 0.5)
                    if full:
                        S = w[t, h * dk:(h + 1) * dk, None] * S - torch.outer(p[t, h * dk:(h + 1) * dk], S.T @ z[t, h * dk:(h + 1) * dk]) \
                            + torch.outer(kk, v[t, h * dv:(h + 1) * dv])
                    else:
                        S = wh[h] * S + torch.outer(kk, v[t, h * dv:(h + 1) * dv])
                    want[t, h] = S.T @ q[t, kh * dk:(kh + 1) * dk]
                end[(slot, h)] = S
        for lanes in ((0,) if device == "cpu" else (0, 4, 16)):
            for qdt in (dtype, torch.float32):          # operands in the activation dtype, and as the f32 the operand kernels write
                state = S0.float().to(device).clone()
                f = lambda t: t.float().to(device)      # noqa: E731
                c = lambda t: t.to(qdt).to(device)      # noqa: E731
                got = ops.delta_scan(c(q), c(k), c(v), f(w) if full else None, f(p) if full else None, f(z) if full else None, state, cu,
                                     slots, pos, H, Hk, dk, dv, w_head=None if full else f(wh), k_scale=1.0 if full else 0.5, max_len=19,
                                     lanes=lanes)
                assert rel_err(got.view(T, H, dv), want) < 2e-5, (full, lanes, qdt)
                for (slot, h), S in end.items():
                    assert rel_err(state[slot, h], S) < 2e-5
                assert torch.equal(state[1].cpu(), S0[1].float())      # a slot no sequence holds is not touched


# ---------------------------------------------------------------------------- attention: mask edges, sink, far keys
def attend(q, k, v, qpos, hscale, first, sink=True):
    """Plain softmax with one more term of score 0 in the denominator: q [H, d] at position qpos over
    keys first(qpos) .. qpos of k [n, G, d], v [n, G, dv] (float64)."""
    H, G = q.shape[0], k.shape[1]
    out = torch.zeros(H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        kv = h // (H // G)
        lo = first(qpos)
        s = (k[lo:qpos + 1, kv] @ q[h]) * float(hscale[h])
        e = torch.exp(s)
        out[h] = (e[:, None] * v[lo:qpos + 1, kv]).sum(0) / ((1.0 if sink else 0.0) + e.sum())
    return out


def paged(k, v, table, device, dtype, nblocks):
    n, G, d = k.shape
    kc = torch.zeros(nblocks, G, BS, d, dtype=dtype, device=device)
    vc = torch.zeros(nblocks, G, v.shape[2], BS, dtype=dtype, device=device)
    for j in range(n):
        kc[table[j // BS], :, j % BS] = k[j].to(dtype).to(device)
        vc[table[j // BS], :, :, j % BS] = v[j].to(dtype).to(device)
    return kc, vc


def run_attention(q, k, v, hscale, mkind, msize, sink, start, device, dtype, splits=(1,)):
    """Queries q [n, H, d] at positions start .. start + n - 1 over cached keys 0 .. start + n - 1: as one
    prompt portion and as n decode rows (each with every number of key splits in ``splits``)."""
    n, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    ctx = start + n
    table = list(range(3, 3 + (ctx + BS - 1) // BS))[::-1]
    kc, vc = paged(k[:ctx], v[:ctx], table, device, dtype, 3 + len(table))
    i32 = dict(dtype=torch.int32, device=device)
    bt = torch.tensor([table], **i32)
    hs = hscale.float().to(device)
    qq = q.reshape(n, H * d).to(dtype).to(device)
    out = torch.zeros(n, H * dv, dtype=dtype, device=device)
    ops.sink_attention_prefill(qq, kc, vc, bt, torch.tensor([0, n], **i32), torch.tensor([ctx], **i32), H, G, d, dv, hs, mkind, msize,
                               sink, None, 0, out, q_lens_cpu=[n])
    res = [out.float().cpu().view(n, H, dv)]
    for Z in splits:
        dec = torch.zeros(n, H * dv, dtype=dtype, device=device)
        ops.sink_attention_decode(qq, kc, vc, bt.expand(n, -1).contiguous(), torch.arange(start + 1, ctx + 1, **i32), H, G, d, dv, hs,
                                  mkind, msize, sink, None, 0, dec, splits=Z)
        res.append(dec.float().cpu().view(n, H, dv))
    return res


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("size", [5, 16, 23, 64, 530])   # 530: the prefill kernel's form for long key ranges
def test_chunk_edges_in_prompts_and_in_decoding(size, device, dtype):
    """One key per chunk is made to stand out (its score towers over the rest).  A query in the same chunk
    returns that key's value; a query one position past the chunk's end must not see it, whatever page
    or 32-key step the edge falls into; the query that IS the first key of a chunk sees only itself."""
    g = torch.Generator().manual_seed(size)
    n, H, G, d, dv = (150 if size < 100 else 570), 2, 1, 16, 8
    k, v, q = q16(rnd(g, n, G, d, scale=0.1)), q16(rnd(g, n, G, dv)), q16(rnd(g, n, H, d, scale=0.1))
    big = torch.zeros(d, dtype=torch.float64)
    big[3] = 8.0
    for c0 in range(0, n, size):
        k[c0, 0] = big                         # the first key of every chunk stands out ...
    q[:, :, 3] = 4.0                           # ... for every query
    hscale = torch.tensor([1.0, 0.5], dtype=torch.float64)
    first = lambda p: (p // size) * size       # noqa: E731
    want = torch.stack([attend(q[i], k, v, i, hscale, first) for i in range(n)])
    for start in (0, 37):                      # a portion that starts inside a chunk, too
        for got in run_attention(q[start:], k, v, hscale, ops.MASK_CHUNK, size, True, start, device, dtype, splits=(1, 3)):
            assert rel_err(got, want[start:]) < tol(dtype), (size, start)
    # what the test is about: inside the chunk the marked key takes (almost) all the weight
    i = min(size - 1, n - 1)
    assert rel_err(want[i, 0], v[0, 0]) < 0.05 or size == 1


@pytest.mark.parametrize("device,dtype", ALL)
def test_far_key_window_and_plain_causal(device, dtype):
    """A key 400 positions back among hundreds of small ones, under the plain causal mask (seen), under a
    sliding window of 400 (just outside) and of 401 (just inside); key splits of the decode kernel."""
    g = torch.Generator().manual_seed(11)
    n, H, G, d, dv = 470, 4, 2, 32, 24
    k, v, q = q16(rnd(g, n, G, d, scale=0.05)), q16(rnd(g, n, G, dv)), q16(rnd(g, n, H, d, scale=0.05))
    k[50, :, 7] = 6.0
    q[450:, :, 7] = 5.0
    hscale = torch.tensor([0.5, 0.4, 0.3, 0.45], dtype=torch.float64)
    for mkind, msize, first in ((ops.MASK_CAUSAL, 0, lambda p: 0), (ops.MASK_WINDOW, 400, lambda p: max(0, p - 399)),
                                (ops.MASK_WINDOW, 401, lambda p: max(0, p - 400))):
        want = torch.stack([attend(q[i], k, v, i, hscale, first) for i in range(440, n)])
        for got in run_attention(q[440:], k, v, hscale, mkind, msize, True, 440, device, dtype, splits=(1, 2, 5)):
            assert rel_err(got, want) < tol(dtype), (mkind, msize)
    # position 450 is the first whose window of 401 holds key 50, and the last whose window of 400 ... does not
    a = attend(q[450], k, v, 450, hscale, lambda p: max(0, p - 400))
    b = attend(q[450], k, v, 450, hscale, lambda p: max(0, p - 399))
    assert float((a - b).abs().max()) > 0.1


@pytest.mark.parametrize("device,dtype", ALL)
def test_sink_takes_the_weight_of_low_scores(device, dtype):
    """Scores far below zero leave the output near zero (the sink holds the weight), scores far above zero
    make the sink irrelevant, and without a sink the weights sum to one in both cases."""
    g = torch.Generator().manual_seed(12)
    n, H, G, d, dv = 40, 2, 2, 16, 16
    k, v = q16(rnd(g, n, G, d)), q16(rnd(g, n, G, dv))
    q = q16(rnd(g, n, H, d))
    first = lambda p: 0   # noqa: E731
    for scale, sink in ((1.0, True), (1.0, False), (-30.0, True), (30.0, True)):
        kk = k.clone()
        if abs(scale) > 1:          # every score = scale * |q|^2-ish: all very low or all very high
            kk = q.mean(1, keepdim=True).expand(n, G, d).clone()
        hscale = torch.tensor([scale / d, scale / d], dtype=torch.float64)
        want = torch.stack([attend(q[i], kk, v, i, hscale, first, sink) for i in range(n)])
        for got in run_attention(q, kk, v, hscale, ops.MASK_CAUSAL, 0, sink, 0, device, dtype):
            assert float((got.double() - want).abs().max()) < tol(dtype) * max(1.0, float(want.abs().max())), (scale, sink)


@pytest.mark.parametrize("device,dtype", ALL)
def test_norm_rotation_and_cache_write(device, dtype):
    """q / k RMS norm with a shared weight, rotation of the first ``rot`` dimensions in the half-split
    pairing at the row's position, unit-RMS values, filed at scattered cache slots."""
    g = torch.Generator().manual_seed(13)
    T, H, G, d, dv, rot, eps = 9, 3, 1, 24, 16, 10, 1e-4
    x = q16(rnd(g, T, (H + G) * d + G * dv + 5))
    qw, kw = q16(rnd(g, d, scale=0.3)) + 1.0, q16(rnd(g, d, scale=0.3)) + 1.0
    pos = torch.tensor([0, 1, 2, 3, 700, 701, 15, 16, 17], dtype=torch.int32)
    slots = torch.tensor([5, 6, 7, 40, 41, -1, 16, 17, 33], dtype=torch.int32)
    inv = torch.tensor([100.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64)
    kc = torch.zeros(4, G, BS, d, dtype=dtype, device=device)
    vc = torch.zeros(4, G, dv, BS, dtype=dtype, device=device)
    xx = x.to(dtype).to(device).clone()
    ops.normrope_kv_write(xx, H, G, d, dv, qw.float().to(device), kw.float().to(device), rot, inv.float().to(device), pos.to(device),
                          eps, kc, vc, slots.to(device))

    def prep(a, w, p):
        a = O.rms_unit(a, eps) * w
        y = a.clone()
        for i in range(rot // 2):
            ang = p * float(inv[i])
            y[..., i] = a[..., i] * math.cos(ang) - a[..., i + rot // 2] * math.sin(ang)
            y[..., i + rot // 2] = a[..., i + rot // 2] * math.cos(ang) + a[..., i] * math.sin(ang)
        return y

    t32 = 2e-4 if dtype == torch.float32 else tol(dtype)    # the angle itself is an f32 product at position 700
    for t in range(T):
        wq = prep(x[t, :H * d].view(H, d), qw, int(pos[t]))
        assert rel_err(xx[t, :H * d].view(H, d), wq) < t32
        if int(slots[t]) >= 0:
            b, o = int(slots[t]) // BS, int(slots[t]) % BS
            assert rel_err(kc[b, :, o], prep(x[t, H * d:(H + G) * d].view(G, d), kw, int(pos[t]))) < t32
            assert rel_err(vc[b, :, :, o], O.rms_unit(x[t, (H + G) * d:(H + G) * d + G * dv].view(G, dv), eps)) < t32
    assert torch.equal(xx[:, (H + G) * d:].float().cpu(), x[:, (H + G) * d:].to(dtype).float())   # v and the rest stay
    assert int((kc.float().abs().sum((1, 3)) > 0).sum()) == 8      # the row whose slot is -1 files nothing


# ---------------------------------------------------------------------------- stream and feed-forward
@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("W", [40, 1030, 4100])
def test_stream_layernorm_and_activation(W, device, dtype):
    g = torch.Generator().manual_seed(W)
    T, eps, alpha = 7, 1e-5, 1.7
    x0, w, b, ls = rnd(g, T, W).float().double(), q16(rnd(g, W, scale=0.2)) + 1, q16(rnd(g, W, scale=0.2)), q16(rnd(g, W, scale=0.3)) + 1
    y = q16(rnd(g, T, W))
    f = lambda t: t.float().to(device)   # noqa: E731
    x = f(x0)
    h = ops.stream_layernorm(x, y.to(dtype).to(device), f(ls), alpha, f(w), f(b), eps, dtype)
    want = O.layer_norm(alpha * x0 + ls * y, w, b, eps)
    assert x.dtype == torch.float32 and rel_err(x, want) < 1e-5 and rel_err(h, want) < tol(dtype) / 4 and h.dtype == dtype
    yf = rnd(g, T, W).float()
    x = f(x0)
    ops.stream_layernorm(x, yf.to(device), f(ls), alpha, f(w), f(b), eps, dtype)        # an f32 branch result
    assert rel_err(x, O.layer_norm(alpha * x0 + ls * yf.double(), w, b, eps)) < 1e-5
    idx = torch.tensor([6, 0, 3], device=device)
    x = f(x0)
    hh = ops.stream_layernorm(x, None, None, 1.0, f(w), f(b), eps, dtype, idx=idx)      # rows for the LM head: x untouched
    assert torch.equal(x.cpu(), x0.float()) and rel_err(hh, O.layer_norm(x0, w, b, eps)[idx.cpu()]) < tol(dtype) / 4
    gu = q16(rnd(g, T, 2 * 36, scale=2.0))
    got = ops.gelu_tanh_mul(gu.to(dtype).to(device))
    assert rel_err(got, O.gelu_tanh(gu[:, :36]) * gu[:, 36:]) < tol(dtype) / 2
    a, c = q16(rnd(g, T, W)), q16(rnd(g, T, W, scale=3.0))
    got = ops.dual_rmsnorm_mean(a.to(dtype).to(device), f(w), c.to(dtype).to(device), f(ls), eps)
    assert got.dtype == torch.float32 and rel_err(got, 0.5 * (O.rms_unit(a, eps) * w + O.rms_unit(c, eps) * ls)) < 1e-5
    tok = q16(rnd(g, 13, W))
    ids = torch.tensor([3, 12, 0, 3], dtype=torch.int32, device=device)
    xs, hs = ops.embed_stream(ids, tok.to(dtype).to(device), dtype)
    assert xs.dtype == torch.float32 and hs.dtype == dtype and rel_err(xs, tok[ids.cpu().long()]) == 0 and rel_err(hs, tok[ids.cpu().long()]) == 0
