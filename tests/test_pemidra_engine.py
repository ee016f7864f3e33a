"""The Pemidra decoder through the framework's engine (model registry, loader, runner, paged cache, state
slots, scheduler, hipGraph decode, replay and generation entry points) against the plain float64 forward
of ``pemidra_oracle``.  Small random models of several shapes; CPU path and (``gpu`` marker) HIP kernels
in f32 and bf16."""
import io
import json

import pytest
import torch

import pemidra_oracle as O
from llm_kubernetes_minikube_sharp4dev_amd.engine.llm_engine import LLMEngine
from llm_kubernetes_minikube_sharp4dev_amd.engine.sampling import SamplingParams
from llm_kubernetes_minikube_sharp4dev_amd.models import PemidraConfig, PemidraModel, build_decoder, load_decoder_dir

CPU32 = pytest.param("cpu", torch.float32, id="cpu-f32")
GPU32 = pytest.param("cuda", torch.float32, id="gpu-f32", marks=pytest.mark.gpu)
GPU16 = pytest.param("cuda", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)
ALL = [CPU32, GPU32, GPU16]


def ret(heads, dim, vdim, decay):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def gen(heads, dim, lora):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim, "lora": lora}}


def par(heads, kv, dim, vdim, scale, size, rot, base, rh, rkv, rdim, rvdim, conv, la, lg):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size},
                 "rot": {"dims": rot, "base": base}},
        "right": {"heads": rh, "kv_heads": rkv, "dim": rdim, "vdim": rvdim, "conv": conv, "lora_a": la, "lora_g": lg}}}


def ff(layer, n):
    return dict(layer, mlp={"kind": "dense", "ff": n} if n else None)


def config(layers, width, vocab=97, alpha=1.5, eps=1e-5):
    return {"architecture": "Pemidra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha, "layers": layers}


CONFIGS = {
    # all three mixers, GQA 2:1 on both sides of the parallel layer, a chunk of 12 positions, feed-forward on two layers
    "three": config([ff(gen(2, 16, 6), 0), ff(ret(2, 16, 24, [0.9, 0.97]), 80),
                     ff(par(4, 2, 32, 16, 0.2, 12, 16, 100.0, 4, 2, 16, 8, 3, 5, 7), 96)], 64),
    # the parallel layer first and without a feed-forward, alpha 1, one head / one kv head, a decay of 1, full rotation,
    # a chunk of 7 (never a page's size), two taps, sizes that are multiples of nothing convenient
    "odd": config([ff(par(3, 1, 20, 12, 0.3, 7, 20, 1000.0, 3, 3, 10, 14, 2, 3, 4), 0), ff(ret(1, 12, 12, [1.0]), 50),
                   ff(gen(3, 10, 2), 50)], 36, vocab=61, alpha=1.0, eps=1e-6),
    # a chunk longer than any test sequence (plain causal inside), a long convolution, wide key heads, no rotation at all
    "wide": config([ff(ret(2, 72, 40, [0.99, 0.8]), 0), ff(par(2, 2, 40, 48, 0.15, 4096, 0, 10000.0, 2, 1, 24, 40, 7, 8, 8), 64),
                    ff(gen(1, 136, 9), 0)], 56, vocab=130, alpha=2.5),
    # projections the MFMA / weight-streaming kernels tile: no vendor GEMM, decode steps captured in hipGraphs
    "mid": config([ff(ret(4, 64, 64, [0.99, 0.98, 0.96, 0.9]), 0), ff(par(4, 2, 64, 64, 0.125, 48, 32, 10000.0, 4, 2, 64, 64, 4, 128, 128), 512),
                   ff(gen(4, 64, 128), 0)], 256, vocab=512),
}
_models = {}


def model_and_weights(name, device, dtype, seed=3):
    key = (name, device, dtype)
    if key not in _models:
        m = build_decoder(PemidraConfig.from_json(CONFIGS[name], name), device=device, dtype=dtype, seed=seed)
        _models[key] = (m, {k: v.cpu() for k, v in m.native_state_dict().items()})
    return _models[key]


def engine(m, tokens=512, seqs=4, **kw):
    return LLMEngine(m, None, block_size=16, max_model_len=tokens, max_num_seqs=seqs, num_blocks=-(-tokens // 16), eos_ids=set(), **kw)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, want, dtype):
    """f32: every position within 1e-4 of the oracle.  bf16: the first tokens of a sequence are ill-conditioned
    in any 16-bit run of this design (a read-out of a state that holds one or two writes is a near-zero dot
    product times a value, and the per-head unit norm blows its rounding -- even its sign -- up to order one),
    so half of the positions must be within 3e-2 and none may be further off than half the logits' range;
    the f32 runs of the same kernels carry the sharp comparison."""
    want = want.double()
    err = (got.double().cpu() - want).abs().reshape(want.shape[0], -1).amax(1) / want.abs().max()
    if dtype == torch.float32:
        return float(err.max()) < 1e-4, float(err.max())
    return float(err.median()) < 3e-2 and float(err.max()) < 0.5, (float(err.median()), float(err.max()))


def replay(eng, rid, tokens, cuts, end=True):
    """Feed ``tokens`` in portions of the sizes ``cuts`` (the rest one by one); logits of every position."""
    out, at = [], 0
    sizes = list(cuts)
    while at < len(tokens):
        n = min(sizes.pop(0) if sizes else 1, len(tokens) - at)
        last = at + n == len(tokens)
        out.append(eng.replay_step([(rid, tokens[at:at + n], list(range(n)))], [rid] if last and end else []))
        at += n
    return torch.cat(out)


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_streams_and_logits(name, device, dtype):
    m, sd = model_and_weights(name, device, dtype)
    t = toks(45, m.cfg.vocab_size, 1)
    streams = []
    want = O.forward(CONFIGS[name], sd, t, streams)
    eng = engine(m)
    from llm_kubernetes_minikube_sharp4dev_amd.engine.sequence import Sequence
    sq = Sequence(list(t), SamplingParams(max_tokens=1))
    assert eng.scheduler.admit_forced(sq, len(t))
    si, _ = eng.runner.prepare([(sq, 0, len(t))], want={id(sq): list(range(len(t)))})
    ids, meta = eng.runner._meta(si)
    taps = []
    with torch.inference_mode():
        m(ids, meta, eng.runner.kv_caches, taps=taps)
    eng.scheduler.finish(sq, "stop")
    assert len(taps) == len(streams) == m.cfg.num_layers
    for r, (a, b) in enumerate(zip(taps, streams)):     # the f32 stream after every layer
        ok, err = close(a, b, dtype)
        assert ok, (r, err)
    ok, err = close(replay(eng, "w", t, [len(t)]), want, dtype)
    assert ok, err


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("name", ["three", "odd"])
def test_prefill_equals_token_by_token_and_portions(name, device, dtype):
    """One step for the whole prompt, one token per step, and portions of changing size down to two tokens
    (cut inside pages and inside chunks) give the same logits at every position."""
    m, sd = model_and_weights(name, device, dtype)
    t = toks(70, m.cfg.vocab_size, 2)
    want = O.forward(CONFIGS[name], sd, t)
    eng = engine(m)
    for cuts in ([70], [], [1, 2, 2, 3, 16, 17, 5, 2], [33, 2, 31], [6, 7, 8]):
        ok, err = close(replay(eng, "r", t, cuts), want, dtype)
        assert ok, (cuts, err)


@pytest.mark.parametrize("device,dtype", ALL)
def test_mixed_batches_equal_each_request_alone(device, dtype):
    """Five requests of unequal lengths share steps: portions of some beside single tokens of others, a
    request sitting out steps, requests ending and a new one taking the freed pages and slot."""
    name = "three"
    m, sd = model_and_weights(name, device, dtype)
    V = m.cfg.vocab_size
    T = {"a": toks(60, V, 10), "b": toks(21, V, 11), "c": toks(9, V, 12), "d": toks(40, V, 13), "e": toks(33, V, 14)}
    want = {k: O.forward(CONFIGS[name], sd, v) for k, v in T.items()}
    plan = [[("a", 17)], [("a", 15), ("b", 20), ("c", 1)], [("a", 1), ("b", 1), ("c", 2), ("d", 31)],
            [("a", 1), ("c", 6), ("d", 1)], [("a", 26), ("d", 1)], [("d", 7), ("e", 2)], [("e", 30)], [("e", 1)]]
    eng = engine(m, tokens=160, seqs=4)   # a + b + c + d live together need 64 + 32 + 16 + 48 tokens of pages
    at = {k: 0 for k in T}
    got = {k: [] for k in T}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, T[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(T[k]):
                end.append(k)
        lg = eng.replay_step(entries, end)
        r = 0
        for k, n in step:
            got[k].append(lg[r:r + n])
            r += n
    assert at == {k: len(v) for k, v in T.items()}
    assert eng.allocator.num_free == eng.runner.num_blocks and eng.state_pool.num_free == 4
    for k in T:
        ok, err = close(torch.cat(got[k]), want[k], dtype)
        assert ok, (k, err)
        # the same portions alone, in the same number format: nothing but rounding may separate the two runs
        alone = replay(eng, k + "-alone", T[k], [n for step in plan for kk, n in step if kk == k])
        d = float((alone.double() - torch.cat(got[k]).double()).abs().max() / want[k].abs().max())
        assert d < (1e-5 if dtype == torch.float32 else 6e-2), (k, d)


@pytest.mark.parametrize("device,dtype", ALL)
def test_freed_pages_and_slots_are_used_again(device, dtype):
    """A pool of exactly one request's size and ONE state slot: every request runs in the pages and the
    slot its predecessor left, and repeats its own first run bit for bit; a second live request is refused."""
    m, sd = model_and_weights("wide", device, dtype)
    V = m.cfg.vocab_size
    a, b = toks(48, V, 20), toks(41, V, 21)
    eng = engine(m, tokens=48, seqs=1)
    first = replay(eng, "a", a, [20, 5])
    other = replay(eng, "b", b, [3, 30])
    again = replay(eng, "a2", a, [20, 5])
    assert torch.equal(first, again)
    assert close(first, O.forward(CONFIGS["wide"], sd, a), dtype)[0]
    assert close(other, O.forward(CONFIGS["wide"], sd, b), dtype)[0]
    eng.replay_step([("x", a[:5], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([("y", b[:5], [])])


@pytest.mark.parametrize("device,dtype", ALL)
def test_long_decode_through_pages_and_chunks(device, dtype):
    """150 single-token steps after a short prompt (across many page and chunk borders), two requests side
    by side."""
    m, sd = model_and_weights("odd", device, dtype)
    V = m.cfg.vocab_size
    a, b = toks(170, V, 30), toks(158, V, 31)
    eng = engine(m, tokens=352, seqs=2)
    ga, gb = [eng.replay_step([("a", a[:20], list(range(20)))])], [eng.replay_step([("b", b[:8], list(range(8)))])]
    for i in range(150):
        lg = eng.replay_step([("a", [a[20 + i]], [0]), ("b", [b[8 + i]], [0])])
        ga.append(lg[:1])
        gb.append(lg[1:])
    for got, t in ((ga, a), (gb, b)):
        ok, err = close(torch.cat(got), O.forward(CONFIGS["odd"], sd, t), dtype)
        assert ok, err


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("name", ["three", "wide"])
def test_greedy_generation_through_the_scheduler(name, device, dtype):
    """``LLMEngine.generate``: the scheduler admits, chunks (a 24-token step budget) and batches three
    prompts; every generated token must be the oracle's argmax for its prefix (or within a near tie)."""
    m, sd = model_and_weights(name, device, dtype)
    V = m.cfg.vocab_size
    prompts = [toks(50, V, 40), toks(7, V, 41), toks(1, V, 42)]
    eng = LLMEngine(m, None, block_size=16, max_model_len=256, max_num_seqs=3, num_blocks=16, eos_ids=set(),
                    max_num_batched_tokens=24)
    seqs = eng.generate(prompts, SamplingParams.greedy(12))
    assert eng.allocator.num_free == 16 and eng.state_pool.num_free == 3
    for p, s in zip(prompts, seqs):
        assert len(s.output_ids) == 12
        full = p + list(s.output_ids)
        lg = O.forward(CONFIGS[name], sd, full[:-1])[len(p) - 1:]
        for i, tid in enumerate(s.output_ids):
            gap = float(lg[i].max() - lg[i, tid])
            assert gap <= (1e-3 if dtype == torch.float32 else 0.25) * float(lg[i].max() - lg[i].min()), (i, gap)


def test_checkpoint_directory_selects_the_model_and_replays(tmp_path):
    """config.json + model.safetensors on disk: the registry picks the class by the architecture name, the
    ranks of the two-layer projections come from the tensors' shapes, the loader checks shapes, and the
    trace command writes the logits it is asked for."""
    import numpy as np
    from safetensors.torch import save_file

    from llm_kubernetes_minikube_sharp4dev_amd.engine.replay import run_trace

    m, sd = model_and_weights("odd", "cpu", torch.float32)
    cfg = json.loads(json.dumps(CONFIGS["odd"]))
    for l in cfg["layers"]:          # a checkpoint's config names no ranks
        for d in (l["mixer"], l["mixer"].get("right", {})):
            for k in ("lora", "lora_a", "lora_g"):
                d.pop(k, None)
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    sd16 = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    save_file(sd16, str(d / "model.safetensors"))
    m2 = load_decoder_dir(str(d), dtype=torch.float32)
    assert isinstance(m2, PemidraModel) and m2.cfg.num_layers == 3
    assert m2.layers[2].mix.spec.lora == 2 and (m2.layers[0].right.spec.lora_a, m2.layers[0].right.spec.lora_g) == (3, 4)
    t = toks(30, 61, 50)
    want = O.forward(cfg, sd16, t)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": t[:19], "want": [0, 18]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": t[19:20], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": t[20:], "want": [9]}, {"id": "p", "tokens": t[:4], "want": [3]}],
              "end": ["q", "p"]}]
    out = io.StringIO()
    assert run_trace(str(d), "float32", str(tmp_path / "o"), 64, lines=[json.dumps(s) for s in steps], out=out, device="cpu") == 0
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    l0 = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4")).view(2, 61)
    l2 = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4")).view(2, 61)
    assert not (tmp_path / "o" / "1.f32").exists()
    assert close(l0, want[[0, 18]], torch.float32)[0] and close(l2, want[[29, 3]], torch.float32)[0]
    bad = dict(sd16)
    bad["l1.mix.q"] = bad["l1.mix.q"][:-1]
    with pytest.raises(ValueError):
        PemidraModel(m2.cfg, dtype=torch.float32).load_state_dict_native(bad)


@pytest.mark.gpu
def test_captured_decode_graph_matches_the_oracle():
    """bf16 on the GPU with sizes the framework's own GEMM kernels tile: decode steps replay a captured
    hipGraph (state slots and block tables in its static buffers); prompt portions, then 60 single tokens
    (past a chunk's end) for two requests that start at different times, against the float64 forward."""
    m, sd = model_and_weights("mid", "cuda", torch.bfloat16)
    V = m.cfg.vocab_size
    a, b = toks(110, V, 60), toks(95, V, 61)
    wa, wb = O.forward(CONFIGS["mid"], sd, a), O.forward(CONFIGS["mid"], sd, b)
    eng = engine(m, tokens=256, seqs=2)
    ga = [eng.replay_step([("a", a[:33], list(range(33)))]), eng.replay_step([("a", a[33:50], list(range(17)))])]
    gb = []
    for i in range(60):
        entries = [("a", [a[50 + i]], [0])]
        if i == 5:
            entries.append(("b", b[:35], list(range(35))))
        elif i > 5:
            entries.append(("b", [b[35 + i - 6]], [0]))
        lg = eng.replay_step(entries)
        ga.append(lg[:1])
        if i >= 5:
            gb.append(lg[1:])
    captured = [k for k, st in eng.runner.graphs.items() if st.get("graph") is not None]
    assert captured, "no decode bucket was captured"
    for got, want, n in ((ga, wa, 110), (gb, wb, 35 + 54)):
        ok, err = close(torch.cat(got), want[:n], torch.bfloat16)
        assert ok, err


def test_served_through_the_model_manager(tmp_path):
    """The serving stack's model manager builds the preset, wraps it in an engine with state slots and
    prefix caching off, and generates through the server's pipelined step loop; a checkpoint directory
    given for a served name brings its own config."""
    import asyncio

    from safetensors.torch import save_file

    from llm_kubernetes_minikube_sharp4dev_amd.config import Config
    from llm_kubernetes_minikube_sharp4dev_amd.serving.model_manager import ModelManager

    cfg = Config()
    cfg.engine.dtype, cfg.engine.max_num_seqs, cfg.engine.max_model_len = "float32", 4, 256
    mgr = ModelManager(cfg, device="cpu", engine_overrides={"num_blocks": 32})
    h = mgr.generator("pemidra-tiny")
    eng = h.engine
    assert isinstance(eng.model, PemidraModel) and eng.state_pool.num_slots == 4 and not eng.allocator.prefix_caching

    async def both():
        return await asyncio.gather(h.async_engine.generate([5, 6, 7, 8, 9, 10, 11], SamplingParams.greedy(5)),
                                    h.async_engine.generate([3], SamplingParams.greedy(5)))

    try:
        seqs = asyncio.run(both())
    finally:
        h.async_engine.shutdown()
    assert [len(s.output_ids) for s in seqs] == [5, 5]
    assert eng.state_pool.num_free == 4
    sd = {k: v.cpu() for k, v in eng.model.native_state_dict().items()}
    for prompt, sq in zip(([5, 6, 7, 8, 9, 10, 11], [3]), seqs):
        full = prompt + list(sq.output_ids)
        lg = O.forward(eng.model.cfg.to_json(), sd, full[:-1])[len(prompt) - 1:]
        assert [int(x) for x in lg.argmax(-1)] == list(sq.output_ids)
    _, sd_odd = model_and_weights("odd", "cpu", torch.float32)
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(CONFIGS["odd"]))
    save_file({k: v.to(torch.bfloat16) for k, v in sd_odd.items()}, str(d / "model.safetensors"))
    mgr2 = ModelManager(cfg, device="cpu", checkpoints={"pemidra-tiny": str(d)}, engine_overrides={"num_blocks": 32})
    h2 = mgr2.generator("pemidra-tiny")
    try:
        assert isinstance(h2.engine.model, PemidraModel) and h2.engine.model.cfg.hidden == 36 and h2.engine.model.cfg.vocab_size == 61
    finally:
        h2.async_engine.shutdown()


@pytest.mark.gpu
def test_pipelined_generation_on_captured_graphs():
    """The server's step loop on the GPU in bf16: pipelined steps whose decode inputs are gathered on the
    device from the previous step's ids, decode graphs replayed, three requests of different lengths that
    decode across a chunk's end; every token must be the oracle's argmax for its prefix, or within a near tie."""
    import asyncio

    from llm_kubernetes_minikube_sharp4dev_amd.engine.llm_engine import AsyncLLMEngine

    m, sd = model_and_weights("mid", "cuda", torch.bfloat16)
    V = m.cfg.vocab_size
    prompts = [toks(40, V, 70), toks(3, V, 71), toks(18, V, 72)]
    eng = LLMEngine(m, None, block_size=16, max_model_len=256, max_num_seqs=4, num_blocks=24, eos_ids=set(),
                    max_num_batched_tokens=32)
    aeng = AsyncLLMEngine(eng)

    async def run():
        return await asyncio.gather(*[aeng.generate(p, SamplingParams.greedy(16)) for p in prompts])

    try:
        seqs = asyncio.run(run())
    finally:
        aeng.shutdown()
    assert any(st.get("graph") is not None for st in eng.runner.graphs.values())
    assert eng.state_pool.num_free == 4 and eng.allocator.num_free == 24
    for p, sq in zip(prompts, seqs):
        assert len(sq.output_ids) == 16
        full = p + list(sq.output_ids)
        lg = O.forward(CONFIGS["mid"], sd, full[:-1])[len(p) - 1:]
        for i, tid in enumerate(sq.output_ids):
            gap = float(lg[i].max() - lg[i, tid])
            assert gap <= 0.25 * float(lg[i].max() - lg[i].min()), (i, gap)
