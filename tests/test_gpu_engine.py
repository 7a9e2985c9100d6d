"""The engine against the plain implementation, in float32 and bfloat16:
whole requests; most of a request at once and the last 32 tokens one by one;
portions of changing size; mixed batches with so few pages that they are used
again; long decoding; the first tokens of a sequence."""
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32, H.FP32_TOL), ("bfloat16", torch.bfloat16, H.BF16_TOL)]
LENGTHS = {"A": [1, 7, 33, 100, 128, 45], "B": [5, 64, 130, 17, 256, 90], "C": [3, 150, 65, 300, 129, 40]}


def _requests(name, seed=0):
    cfg = H.CONFIGS[name][0]
    return {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, seed * 100 + i)
            for i, n in enumerate(LENGTHS[name])}


_engines = {}
_plain = {}


def _engine(tmp_path_factory, name, dtype, max_tokens, page_size=16, attention="auto"):
    from infinicore_infer_amd.engine import Engine
    key = (name, dtype, max_tokens, page_size, attention)
    if key not in _engines:
        folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
        _engines[key] = (Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=page_size,
                                         max_requests=8, attention_impl=attention), folder)
    return _engines[key]


def _reference(folder, name, requests, bf16):
    key = (name, bf16, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in _plain:
        _plain[key] = H.plain_logits(H.CONFIGS[name][0], H.load_state_dict(folder), requests, bf16)
    return _plain[key]


MODES = {
    "whole": H.trace_whole,
    "last32": H.trace_last_one_by_one,
    "chunks": H.trace_chunks,
    "mixed": H.trace_mixed,
}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay_modes(tmp_path_factory, name, dname, dtype, tol, mode):
    requests = _requests(name)
    steps, max_tokens = MODES[mode](requests)
    engine, folder = _engine(tmp_path_factory, name, dtype, max_tokens)
    ref = _reference(folder, name, requests, dtype == torch.bfloat16)
    got = H.run_trace(engine, steps)
    assert len(got) == sum(len(t) for t in requests.values())
    worst = H.compare(got, ref, tol, "%s %s %s" % (name, dname, mode))
    print("worst error %.3g at %s (allowed %.3g)" % (worst[0], worst[1], tol))
    engine.cache.check_invariants()
    assert not engine.cache.requests, "every request was ended"
    for g in range(len(engine.groups)):
        assert engine.cache.free_pages(g) == engine.num_pages


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_mixed_reuses_pages(tmp_path_factory, dname, dtype, tol):
    """The mixed trace's pool is smaller than what all requests would need together."""
    requests = _requests("B")
    steps, max_tokens = H.trace_mixed(requests)
    assert max_tokens < sum(H.ceil64(len(t)) for t in requests.values())


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("page_size", [16, 64])
def test_generic_attention_path(tmp_path_factory, dname, dtype, tol, page_size):
    """The general attention kernel alone (tiled kernels off) on the head-size-64 model."""
    requests = _requests("C")
    steps, max_tokens = H.trace_mixed(requests, seed=3)
    engine, folder = _engine(tmp_path_factory, "C", dtype, max_tokens, page_size=page_size, attention="generic")
    ref = _reference(folder, "C", requests, dtype == torch.bfloat16)
    H.compare(H.run_trace(engine, steps), ref, tol, "C %s generic page %d" % (dname, page_size))


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_long_decoding(tmp_path_factory, dname, dtype, tol):
    """A short prompt, then every further token one by one up to the model's last position."""
    cfg = H.CONFIGS["C"][0]
    toks = H.random_tokens(cfg["vocab_size"], cfg["max_position_embeddings"], 77)
    requests = {"long": toks}
    steps, max_tokens = H.trace_last_one_by_one(requests, tail=len(toks) - 5)
    engine, folder = _engine(tmp_path_factory, "C", dtype, max_tokens)
    ref = _reference(folder, "C", requests, dtype == torch.bfloat16)
    H.compare(H.run_trace(engine, steps), ref, tol, "C %s long decoding" % dname)


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(tmp_path_factory, name, dname, dtype, tol):
    """Positions 0, 1, 2 fed one by one, and as one portion: the start of a sequence."""
    cfg = H.CONFIGS[name][0]
    toks = H.random_tokens(cfg["vocab_size"], 3, 5)
    engine, folder = _engine(tmp_path_factory, name, dtype, 64)
    ref = _reference(folder, name, {"f": toks}, dtype == torch.bfloat16)
    one = [{"step": i, "entries": [{"id": "f", "tokens": [toks[i]], "want": [0]}], "end": ["f"] if i == 2 else []}
           for i in range(3)]
    H.compare(H.run_trace(engine, one), ref, tol, "first tokens one by one")
    whole = [{"step": 0, "entries": [{"id": "f", "tokens": toks, "want": [0, 1, 2]}], "end": ["f"]}]
    H.compare(H.run_trace(engine, whole), ref, tol, "first tokens as one portion")


def test_out_of_pages_changes_nothing(tmp_path_factory):
    from infinicore_infer_amd.cache import OutOfPages
    from infinicore_infer_amd.engine import StepEntry
    engine, _ = _engine(tmp_path_factory, "A", torch.float32, 64)
    toks = H.random_tokens(256, 60, 1)
    engine.step([StepEntry("x", toks, [])])
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("x", [1], [0]), StepEntry("y", toks[:20], [])])
    assert engine.length("x") == 60 and not engine.has_request("y")
    engine.cache.check_invariants()
    engine.free("x")


def test_bad_tokens_are_refused(tmp_path_factory):
    from infinicore_infer_amd.engine import StepEntry
    engine, _ = _engine(tmp_path_factory, "A", torch.float32, 64)
    with pytest.raises(ValueError):
        engine.step([StepEntry("z", [256], [0])])
    with pytest.raises(ValueError):
        engine.step([StepEntry("z", [1, 2], [2])])
    assert not engine.has_request("z")
