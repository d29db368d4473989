"""The hybrid decoder (Pugovik) through the engine against the plain oracle
(tests/hybrid_oracle.py). Every test makes its own small configuration and
random checkpoint, writes it as a model folder, and loads it with
LLMEngine(folder): config reader, safetensors loader, cache/state managers,
batching and kernels are all the product's. CPU path always; the HIP path
(fp32 and bf16, decode through captured graphs) under the gpu marker."""
import functools
import math

import pytest
import torch

from hybrid_oracle import (as_f64, lat_layer, lin_layer, make_config,
                           make_weights, moe, o_forward, rel_err,
                           write_model_dir)
from xllm_service_amd.engine.engine import LLMEngine
from xllm_service_amd.engine.sampling import SamplingParams

TARGETS = [("cpu", torch.float32),
           pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
           pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]


def _variants():
    m = moe()
    return {
        # the usual shape: linear, linear, attention, attention-sharing
        "mixed": make_config(layers=[
            lin_layer(mlp=m), lin_layer(mlp=m), lat_layer(mlp=m),
            lat_layer(kv_from=2, mlp=m)]),
        # attention first; borrowed latent from a non-adjacent layer; a layer
        # without feed-forward; partial rotation; no frequency scaling
        "attn_first": make_config(width=40, groups=1, mult=1.0, layers=[
            lat_layer(heads=1, dim=6, rot_dim=6, vdim=7, kv_rank=9, dims=4,
                      scaling=False, mlp=moe(4, 1, 8, 0)),
            lin_layer(heads=1, dim=5, vdim=5, decay=[1.0], mlp=None),
            lat_layer(heads=3, dim=6, rot_dim=6, vdim=4, kv_rank=9, dims=4,
                      scaling=False, kv_from=0, mlp=moe(4, 4, 8, 2, 2)),
            lat_layer(heads=2, dim=16, rot_dim=2, vdim=16, kv_rank=70,
                      mlp=moe(8, 2, 8, 4, 1))]),
        # only recurrent layers, many groups, wide values
        "linear_only": make_config(width=64, groups=8, mult=0.25, layers=[
            lin_layer(heads=4, dim=16, vdim=24, mlp=moe(5, 2, 12, 5, 3)),
            lin_layer(heads=2, dim=40, vdim=8, mlp=None)]),
        # only attention layers, two latents of their own
        "attn_only": make_config(width=32, groups=2, layers=[
            lat_layer(mlp=None), lat_layer(heads=4, dim=4, rot_dim=4, vdim=6,
                                           kv_rank=8, mlp=m)]),
    }


@functools.lru_cache(maxsize=None)
def _model(name, tmp_root):
    cfg = _variants()[name]
    w = make_weights(cfg, seed=sum(map(ord, name)))
    folder = write_model_dir(f"{tmp_root}/{name}", cfg, w)
    return cfg, as_f64(w), folder


@pytest.fixture(scope="module")
def root(tmp_path_factory):
    return str(tmp_path_factory.mktemp("hybrid_models"))


def _tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


@functools.lru_cache(maxsize=None)
def _oracle(name, tmp_root, n, seed):
    cfg, w, _ = _model(name, tmp_root)
    return o_forward(cfg, w, _tokens(cfg, n, seed))[0]


def _engine(folder, target, blocks=64, slots=4, **kw):
    dev, dt = target
    return LLMEngine(folder, device=dev, dtype=dt, max_num_seqs=slots,
                     state_slots=slots, max_kv_blocks=blocks,
                     max_model_len=blocks * 16, enable_graphs=dev == "cuda",
                     swap_space_mb=0, **kw)


def _check(got, want, target, what=""):
    e = rel_err(got, want)
    if target[1] == torch.float32:
        assert float(e.max()) < 5e-4, (what, float(e.max()))
    else:       # bf16: rounding-sized error; a rare router flip is tolerated
        assert float(e.median()) < 0.06, (what, float(e.median()))
        assert float((e > 0.15).float().mean()) <= 0.1, (what, e)


def _run_portions(eng, rid, toks, cuts, end=True):
    """Feed toks in portions of the given sizes; logits at every position."""
    out, at = [], 0
    for n in cuts:
        last = at + n == len(toks)
        out.append(eng.score_step([(rid, toks[at:at + n], list(range(n)))],
                                  finished=[rid] if (last and end) else []))
        at += n
    assert at == len(toks)
    return torch.cat(out)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "attn_first", "linear_only",
                                  "attn_only"])
def test_whole_prompt(root, target, name):
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    for n, seed in ((1, 1), (2, 2), (67, 3)):   # first tokens, past a tile
        toks = _tokens(cfg, n, seed)
        got = _run_portions(eng, f"w{n}", toks, [n])
        _check(got, _oracle(name, root, n, seed), target, (name, n))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "attn_first"])
def test_layers_residual_stream(root, target, name):
    """Layer by layer: hook the residual after every layer of one prompt."""
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    toks = _tokens(cfg, 21, 5)
    seen = []
    hooks = [l.register_forward_hook(lambda m, i, o: seen.append(
        o.detach().float().cpu().clone())) for l in eng.model.layers]
    eng.score_step([("a", toks, [0])], finished=["a"])
    for h in hooks:
        h.remove()
    trail = o_forward(cfg, w, toks)[1]
    assert len(seen) == len(trail)
    for i, (a, b) in enumerate(zip(seen, trail)):
        # per token. In bf16 the router sees a rounded input, so a token
        # whose expert scores nearly tie takes another expert and differs
        # from there on: the median is the bf16 criterion, the fp32 run is
        # the strict one
        err = ((a.double() - b).norm(dim=-1) / b.norm(dim=-1))
        if target[1] == torch.float32:
            assert float(err.max()) < 2e-4, (name, i, float(err.max()))
        else:
            assert float(err.median()) < 0.1, (name, i, err)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "attn_first", "linear_only"])
def test_prefill_then_token_by_token(root, target, name):
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    n = 40
    toks = _tokens(cfg, n, 7)
    want = _oracle(name, root, n, 7)
    for first in (1, 15, 16, 17):
        got = _run_portions(eng, f"d{first}", toks, [first] + [1] * (n - first))
        _check(got, want, target, (name, first))


@pytest.mark.parametrize("target", TARGETS)
def test_portions_of_many_sizes(root, target):
    cfg, w, folder = _model("mixed", root)
    eng = _engine(folder, target)
    n = 150
    toks = _tokens(cfg, n, 8)
    want = _oracle("mixed", root, n, 8)
    for cuts in ([2] * 10 + [16, 15, 17, 2, 64, 3, 1, 1, 11],
                 [63, 2, 64, 1, 2, 2, 16],
                 [65, 31, 33, 1, 1, 17, 2]):
        assert sum(cuts) == n
        got = _run_portions(eng, "p", toks, cuts)
        _check(got, want, target, cuts)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "attn_first"])
def test_long_decoding_across_pages(root, target, name):
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    n = 120
    toks = _tokens(cfg, n, 9)
    got = _run_portions(eng, "l", toks, [9] + [1] * (n - 9))
    _check(got, _oracle(name, root, n, 9), target, name)


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_batch_with_reused_pages_and_slots(root, target):
    """Three slots and a pool far smaller than the sum of all requests:
    requests come and go in mixed batches (prompt portions beside single
    tokens), later ones land on freed pages and slots that still hold the
    earlier ones' data. Every request must match its own run alone."""
    cfg, w, folder = _model("mixed", root)
    lens = dict(a=70, b=3, c=33, d=50, e=18, f=41)
    toks = {k: _tokens(cfg, n, 20 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: _oracle("mixed", root, n, 20 + i)
            for i, (k, n) in enumerate(lens.items())}
    eng = _engine(folder, target, blocks=10, slots=3)   # 160 tokens of pages
    plan = [
        [("a", 30), ("b", 2)],
        [("a", 1), ("b", 1), ("c", 17)],
        [("a", 16), ("c", 16)],                 # b done: slot + page free
        [("a", 1), ("d", 2)],                   # d reuses b's slot
        [("a", 22), ("d", 1)],                  # a done (70)
        [("d", 31), ("e", 18)],                 # c done earlier; e on a's pages
        [("d", 1), ("f", 5)],
        [("d", 15), ("f", 1)],
        [("f", 35)],
    ]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in plan:
        entries, done = [], []
        for k, n in step:
            entries.append((k, toks[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == lens[k]:
                done.append(k)
        out = eng.score_step(entries, finished=done)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
    assert at == lens
    assert eng.block_manager.num_free == 10
    assert eng.state_manager.num_free == 3
    for k in lens:
        _check(torch.cat(got[k]), want[k], target, k)


@pytest.mark.parametrize("target", TARGETS)
def test_slot_exhaustion_is_refused(root, target):
    cfg, w, folder = _model("linear_only", root)
    eng = _engine(folder, target, slots=2)
    eng.score_step([("a", [1, 2], []), ("b", [3], [])])
    with pytest.raises(RuntimeError):
        eng.score_step([("c", [4], [])])


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_scheduler(root, target):
    """generate(): continuous batching with chunked prompts (a 16-token step
    budget), three unequal prompts on two state slots, greedy sampling.
    The oracle continues each prompt alone; a step whose two best oracle
    logits are closer than the dtype's noise ends the comparison."""
    cfg, w, folder = _model("mixed", root)
    dev, dt = target
    eng = LLMEngine(folder, device=dev, dtype=dt, max_num_seqs=2,
                    state_slots=2, max_kv_blocks=32, max_model_len=256,
                    max_batched_tokens=16, enable_graphs=dev == "cuda",
                    swap_space_mb=0)
    prompts = [_tokens(cfg, n, 40 + n) for n in (37, 5, 20)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    margin = 1e-3 if dt == torch.float32 else 0.15
    for p, out in zip(prompts, outs):
        assert len(out) == 6
        seq = list(p)
        for tok in out:
            top = o_forward(cfg, w, seq)[0][-1].topk(2)
            if float(top.values[0] - top.values[1]) < margin:
                break
            assert tok == int(top.indices[0])
            seq.append(tok)
    assert eng.block_manager.num_free == 32
    assert eng.state_manager.num_free == 2


def test_config_rejects_bad_sharing(tmp_path):
    cfg = make_config(layers=[lat_layer(kv_from=1), lat_layer()])
    folder = write_model_dir(str(tmp_path / "bad"), cfg, {})
    with pytest.raises(ValueError):
        LLMEngine(folder, device="cpu")
