"""The Lebepel decoder through the framework's engine (model registry, loader, runner, paged cache,
state slots, scheduler, hipGraph decode, replay and generation entry points) against the plain
float64 forward of ``hybrid_oracle``.  Small random models of several shapes; CPU path and
(``gpu`` marker) HIP kernels in f32 and bf16."""
import io
import json

import pytest
import torch

import hybrid_oracle as O
from llm_kubernetes_minikube_sharp4dev_amd.engine.llm_engine import LLMEngine
from llm_kubernetes_minikube_sharp4dev_amd.engine.sampling import SamplingParams
from llm_kubernetes_minikube_sharp4dev_amd.models import LebepelConfig, LebepelModel, build_decoder, load_decoder_dir

CPU32 = pytest.param("cpu", torch.float32, id="cpu-f32")
GPU32 = pytest.param("cuda", torch.float32, id="gpu-f32", marks=pytest.mark.gpu)
GPU16 = pytest.param("cuda", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)
ALL = [CPU32, GPU32, GPU16]


def att(heads, kv, dim, vdim, scale):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}}


def ssm(heads, vdim, state, groups, conv, ng):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": ng}}


def ff(layer, n):
    return dict(layer, mlp={"kind": "dense", "ff": n} if n else None)


def config(layers, width, vocab=97, loop=None, mult=0.6, cap=12.0, eps=1e-5, max_pos=512):
    d = {"architecture": "Lebepel", "vocab": vocab, "width": width, "max_positions": max_pos, "norm": {"eps": eps},
         "residual_mult": mult, "logit_softcap": cap, "layers": layers}
    if loop:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


CONFIGS = {
    # looped span in the middle, GQA 2:1, both mixers with a feed-forward
    "loop-mid": config([ff(ssm(4, 16, 16, 2, 4, 2), 96), ff(att(4, 2, 32, 32, 0.18), 96), ff(ssm(4, 16, 16, 2, 4, 2), 0),
                        ff(att(4, 2, 32, 32, 0.18), 96)], 64, loop=(1, 3, 2)),
    # no loop at all, no feed-forward anywhere, one kv head per query head, multiplier 1, no cap, one norm group
    "plain": config([ff(att(2, 2, 16, 48, 0.25), 0), ff(ssm(2, 24, 8, 1, 2, 1), 0)], 48, mult=1.0, cap=0.0, eps=1e-6),
    # the whole stack three times, 8 query heads on one kv head, q/k wider than v, long convolution
    "loop-all": config([ff(att(8, 1, 40, 24, 0.12), 80), ff(ssm(6, 8, 40, 3, 7, 3), 80)], 56, vocab=130, loop=(0, 2, 3),
                       mult=0.4, cap=30.0),
    # sizes that are multiples of nothing convenient
    "odd": config([ff(ssm(3, 10, 12, 1, 3, 1), 50), ff(att(3, 1, 20, 12, 0.3), 50)], 36, vocab=61, loop=(1, 2, 2)),
    # projections the MFMA / weight-streaming kernels tile: no vendor GEMM, decode steps captured in hipGraphs
    "mid": config([ff(att(4, 2, 64, 64, 0.125), 512), ff(ssm(8, 32, 64, 2, 4, 2), 512)], 256, vocab=512, loop=(0, 2, 2),
                  mult=0.5, cap=25.0),
}
_models = {}


def model_and_weights(name, device, dtype, seed=3):
    key = (name, device, dtype)
    if key not in _models:
        m = build_decoder(LebepelConfig.from_json(CONFIGS[name], name), device=device, dtype=dtype, seed=seed)
        _models[key] = (m, {k: v.cpu() for k, v in m.native_state_dict().items()})
    return _models[key]


def engine(m, tokens=512, seqs=4, **kw):
    return LLMEngine(m, None, block_size=16, max_model_len=m.cfg.max_position, max_num_seqs=seqs,
                     num_blocks=-(-tokens // 16), eos_ids=set(), **kw)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, want, dtype):
    want = want.double()
    err = float((got.double().cpu() - want).abs().max() / want.abs().max())
    return err < (1e-4 if dtype == torch.float32 else 5e-2), err


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
    # the f32 stream after every layer run, through the runner's own step inputs
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
    for r, (a, b) in enumerate(zip(taps, streams)):
        ok, err = close(a, b, dtype)
        assert ok, (r, err)
    ok, err = close(replay(eng, "w", t, [len(t)]), want, dtype)
    assert ok, err


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("name", ["loop-mid", "odd"])
def test_prefill_equals_token_by_token_and_portions(name, device, dtype):
    """One step for the whole prompt, one token per step, and portions of 1, 2, 2, 3, 16, 17, 5, 2
    tokens (then single tokens) give the same logits at every position."""
    m, sd = model_and_weights(name, device, dtype)
    t = toks(70, m.cfg.vocab_size, 2)
    want = O.forward(CONFIGS[name], sd, t)
    eng = engine(m)
    for cuts in ([70], [], [1, 2, 2, 3, 16, 17, 5, 2], [33, 2, 31]):
        ok, err = close(replay(eng, "r", t, cuts), want, dtype)
        assert ok, (cuts, err)


@pytest.mark.parametrize("device,dtype", ALL)
def test_mixed_batches_equal_each_request_alone(device, dtype):
    """Four requests of unequal lengths share steps: portions of some beside single tokens of others,
    a request sitting out steps, requests ending and a new one taking the freed pages and slot."""
    name = "loop-mid"
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


@pytest.mark.parametrize("device,dtype", ALL)
def test_freed_pages_and_slots_are_used_again(device, dtype):
    """A pool of exactly one request's size and ONE state slot: every request runs in the pages and
    the slot its predecessor left, and repeats its own first run bit for bit; a second live request
    is refused instead of sharing them."""
    m, sd = model_and_weights("loop-all", device, dtype)
    V = m.cfg.vocab_size
    a, b = toks(48, V, 20), toks(41, V, 21)
    eng = engine(m, tokens=48, seqs=1)
    first = replay(eng, "a", a, [20, 5])
    other = replay(eng, "b", b, [3, 30])
    again = replay(eng, "a2", a, [20, 5])
    assert torch.equal(first, again)
    assert close(first, O.forward(CONFIGS["loop-all"], sd, a), dtype)[0]
    assert close(other, O.forward(CONFIGS["loop-all"], sd, b), dtype)[0]
    eng.replay_step([("x", a[:5], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([("y", b[:5], [])])


@pytest.mark.parametrize("device,dtype", ALL)
def test_long_decode_through_pages(device, dtype):
    """150 single-token steps after a short prompt (across many page borders; on the GPU through
    the captured decode graph), two requests side by side."""
    m, sd = model_and_weights("plain", device, dtype)
    V = m.cfg.vocab_size
    a, b = toks(170, V, 30), toks(158, V, 31)
    eng = engine(m, tokens=352, seqs=2)
    ga, gb = [eng.replay_step([("a", a[:20], list(range(20)))])], [eng.replay_step([("b", b[:8], list(range(8)))])]
    for i in range(150):
        lg = eng.replay_step([("a", [a[20 + i]], [0]), ("b", [b[8 + i]], [0])])
        ga.append(lg[:1])
        gb.append(lg[1:])
    for got, t in ((ga, a), (gb, b)):
        ok, err = close(torch.cat(got), O.forward(CONFIGS["plain"], sd, t), dtype)
        assert ok, err


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("name", ["loop-mid", "plain"])
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
    """config.json + model.safetensors on disk: the registry picks the class by the architecture
    name, the loader checks shapes, and the trace command writes the logits it is asked for."""
    from safetensors.torch import save_file

    from llm_kubernetes_minikube_sharp4dev_amd.engine.replay import run_trace

    m, sd = model_and_weights("odd", "cpu", torch.float32)
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(CONFIGS["odd"]))
    save_file({k: v.to(torch.bfloat16) for k, v in sd.items()}, str(d / "model.safetensors"))
    sd16 = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    m2 = load_decoder_dir(str(d), dtype=torch.float32)
    assert isinstance(m2, LebepelModel) and m2.cfg.num_layers == 3 and m2.cfg.to_json()["loop"] == CONFIGS["odd"]["loop"]
    t = toks(30, 61, 50)
    want = O.forward(CONFIGS["odd"], sd16, t)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": t[:19], "want": [0, 18]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": t[19:20], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": t[20:], "want": [9]}, {"id": "p", "tokens": t[:4], "want": [3]}],
              "end": ["q", "p"]}]
    out = io.StringIO()
    assert run_trace(str(d), "float32", str(tmp_path / "o"), 64, lines=[json.dumps(s) for s in steps], out=out,
                     device="cpu") == 0
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    import numpy as np
    l0 = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4")).view(2, 61)
    l2 = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4")).view(2, 61)
    assert not (tmp_path / "o" / "1.f32").exists()
    assert close(l0, want[[0, 18]], torch.float32)[0] and close(l2, want[[29, 3]], torch.float32)[0]
    bad = dict(sd16)
    bad["l0.mix.in"] = bad["l0.mix.in"][:-1]
    with pytest.raises(ValueError):
        LebepelModel(m2.cfg, dtype=torch.float32).load_state_dict_native(bad)


@pytest.mark.gpu
def test_captured_decode_graph_matches_the_oracle():
    """bf16 on the GPU with sizes the framework's own GEMM kernels tile: decode steps replay a captured
    hipGraph (state slots and block tables in its static buffers); prompt portions, then 40 single
    tokens for two requests that start at different times, against the float64 forward."""
    m, sd = model_and_weights("mid", "cuda", torch.bfloat16)
    V = m.cfg.vocab_size
    a, b = toks(90, V, 60), toks(75, V, 61)
    wa, wb = O.forward(CONFIGS["mid"], sd, a), O.forward(CONFIGS["mid"], sd, b)
    eng = engine(m, tokens=192, seqs=2)
    ga = [eng.replay_step([("a", a[:33], list(range(33)))]), eng.replay_step([("a", a[33:50], list(range(17)))])]
    gb = []
    for i in range(40):
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
    for got, want, n in ((ga, wa, 90), (gb, wb, 35 + 34)):
        ok, err = close(torch.cat(got), want[:n], torch.bfloat16)
        assert ok, err


def test_served_through_the_model_manager():
    """The serving stack's model manager builds the preset (and a checkpoint directory's own config),
    wraps it in an engine with state slots and prefix caching off, and generates through it."""
    from llm_kubernetes_minikube_sharp4dev_amd.config import Config
    from llm_kubernetes_minikube_sharp4dev_amd.serving.model_manager import ModelManager

    cfg = Config()
    cfg.engine.dtype, cfg.engine.max_num_seqs, cfg.engine.max_model_len = "float32", 4, 256
    mgr = ModelManager(cfg, device="cpu", engine_overrides={"num_blocks": 32})
    h = mgr.generator("lebepel-tiny")
    eng = h.engine
    assert isinstance(eng.model, LebepelModel) and eng.state_pool.num_slots == 4 and not eng.allocator.prefix_caching
    import asyncio

    async def both():   # the server's path: background step loop, pipelined steps, two requests in flight
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


@pytest.mark.gpu
def test_pipelined_generation_on_captured_graphs():
    """The server's step loop on the GPU in bf16: pipelined steps whose decode inputs are gathered on the
    device from the previous step's ids, decode graphs replayed, three requests of different lengths;
    every token must be the oracle's argmax for its prefix, or within a near tie."""
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
