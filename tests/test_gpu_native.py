"""The step issued by one native call against the same step issued kernel by kernel from the parts'
Python forward: the logits must be bit-equal, since both launch the same kernels with the same
arguments.  (Each path is compared with the plain implementation elsewhere; the engine's default is
the native one.)"""
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32), ("bfloat16", torch.bfloat16)]
LENGTHS = {"A": [1, 7, 33, 100, 128, 45], "B": [5, 64, 130, 17, 256, 90], "C": [3, 150, 65, 300, 129, 40],
           "D": [2, 200, 31, 384, 64, 129]}


def _pair(folder, dtype, max_tokens, **kw):
    from infinicore_infer_amd.engine import Engine
    a = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, use_native=True, **kw)
    b = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, use_native=False, **kw)
    assert a.native is not None and b.native is None
    return a, b


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dname,dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_native_steps_equal_python_steps_bit_for_bit(tmp_path_factory, name, dname, dtype, graphs):
    from infinicore_infer_amd.engine import StepEntry
    cfg = H.CONFIGS[name][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, i) for i, n in enumerate(LENGTHS[name])}
    for maker in (H.trace_mixed, H.trace_last_one_by_one):
        steps, max_tokens = maker(requests)
        a, b = _pair(folder, dtype, max_tokens, page_size=16, max_requests=8, use_graphs=graphs)
        for rec in steps:
            ents = [StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]]
            la, lb = a.step(ents), b.step(ents)
            assert (la is None) == (lb is None)
            if la is not None:
                assert torch.equal(la, lb), "%s %s step %d: native and Python-issued logits differ" % (name, dname, rec["step"])
            for rid in rec["end"]:
                a.free(rid)
                b.free(rid)
        assert a.native_steps > 0 and b.native_steps == 0
        if graphs:
            assert a.graph_replays == b.graph_replays > 0


def test_native_step_with_many_rows_and_benchmark_shaped_layers(tmp_path_factory):
    """Library products, the unfused kernels and 20 single-token rows beside a prompt portion, on two layers
    of the benchmark's sizes: native and Python-issued steps agree bit for bit."""
    import os
    from infinicore_infer_amd.engine import StepEntry
    from infinicore_infer_amd.weights import write_random_model
    cfg = dict(model_type="minicpm", vocab_size=5003, hidden_size=2304, num_hidden_layers=2, num_attention_heads=36,
               num_key_value_heads=36, intermediate_size=5760, max_position_embeddings=512, rms_norm_eps=1e-5,
               rope_theta=10000.0, scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True,
               eos_token_id=2)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_native_bench_layers")
    write_random_model(folder, cfg, seed=3, std=0.02)
    a, b = _pair(folder, torch.bfloat16, 24 * 512, page_size=64, max_requests=24)
    ids = ["q%d" % i for i in range(20)]
    for eng in (a, b):
        eng.step([StepEntry(r, H.random_tokens(5003, 10 + 9 * i, i), []) for i, r in enumerate(ids)])
    for j in range(3):
        ents = [StepEntry(r, [7 + i + j], [0]) for i, r in enumerate(ids)]
        ents.insert(5, StepEntry("p", H.random_tokens(5003, 150, 50 + j), [0, 149]))
        la, lb = a.step(ents), b.step(ents)
        assert torch.equal(la, lb)
    for n in (1, 3, 16):                     # few rows: the fused epilogues and the split norm
        ents = [StepEntry(r, [11 + i], [0]) for i, r in enumerate(ids[:n])]
        assert torch.equal(a.step(ents), b.step(ents))


def test_models_with_parts_of_their_own_are_stepped_from_python(tmp_path_factory):
    """A part without a native description keeps the whole model on the Python path: nothing changes for it."""
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model, register_part
    from infinicore_infer_amd.parts.swiglu import SwiGLU
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.config.spec import PartSpec
    from infinicore_infer_amd.weights import init_random_weights
    import dataclasses

    @register_part("feed_forward", "swiglu_of_the_test")
    class Mine(SwiGLU):
        def forward(self, h, ctx, tail=None):          # the same arithmetic, but it is not the built-in forward
            return super().forward(h, ctx)

    spec = config_from_dict(H.TINY_A).model_spec()
    layers = [dataclasses.replace(l, feed_forward=PartSpec("swiglu_of_the_test", l.feed_forward.name, l.feed_forward.params))
              for l in spec.layers]
    model = build_model(dataclasses.replace(spec, layers=layers), Runtime(torch.bfloat16, "cuda:0"))
    init_random_weights(model, seed=1)
    eng = Engine(model, max_tokens=128)
    assert eng.native is None
    plain = build_model(spec, Runtime(torch.bfloat16, "cuda:0"))
    init_random_weights(plain, seed=1)
    assert Engine(plain, max_tokens=128).native is not None


def test_the_c_step_function_through_ctypes(tmp_path_factory):
    """ic_decoder_step as a C caller would use it, without the engine's Python around it: host arrays in the
    shape of inferBatch (tokens, req_lens, req_pos, a block table per request), a pinned staging buffer,
    device memory for the integers and the workspace.  Two steps (prompts of three requests; then single
    tokens of two of them beside a portion of the third) against an engine that is fed the same."""
    import ctypes
    import numpy as np
    from infinicore_infer_amd.engine import Engine, StepEntry
    from infinicore_infer_amd.kernels.lib import IcHostBatch, IcStepBatch, get_lib
    cfg = H.CONFIGS["C"][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "C")
    eng = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=1024, page_size=16, max_requests=4)
    ref = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=1024, page_size=16, max_requests=4, use_native=False)
    lib, dec = get_lib(), eng.native._h
    dev = torch.device("cuda:0")
    prompts = [H.random_tokens(cfg["vocab_size"], n, 40 + i) for i, n in enumerate([150, 9, 70])]
    # the caller's own bookkeeping: pages 0.. handed out in order, 16 tokens a page
    tables = [[], [], []]
    next_page = [0]

    def grow(r, length):
        while len(tables[r]) * 16 < length:
            tables[r].append(next_page[0])
            next_page[0] += 1

    staging = torch.empty(1 << 16, dtype=torch.int32, pin_memory=True)
    ints = torch.empty(1 << 16, dtype=torch.int32, device=dev)
    work = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    lib_ws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def c_step(reqs, toks, pos, want):
        lens = [len(t) for t in toks]
        for r, t, p in zip(reqs, toks, pos):
            grow(r, p + len(t))
        tok = np.array([x for t in toks for x in t], dtype=np.int32)
        req_lens, req_pos = np.array(lens, dtype=np.int32), np.array(pos, dtype=np.int32)
        want_count = np.array([len(w) for w in want], dtype=np.int32)
        want_flat = np.array([x for w in want for x in w], dtype=np.int32)
        tabs = [np.array(tables[r], dtype=np.int32) for r in reqs]
        ptrs = (ctypes.c_void_p * len(reqs))(*[t.ctypes.data for t in tabs])
        tlen = np.array([len(t) for t in tabs], dtype=np.int32)
        hb = IcHostBatch(len(tok), len(reqs), tok.ctypes.data, req_lens.ctypes.data, req_pos.ctypes.data,
                         want_count.ctypes.data, want_flat.ctypes.data, ctypes.cast(ptrs, ctypes.c_void_p),
                         tlen.ctypes.data, lib.ic_attn_prefill_tile_rows(), 0)
        n = lib.ic_decoder_step_ints(dec, ctypes.byref(hb))
        assert 0 < n <= staging.numel()
        logits = torch.empty(int(want_count.sum()), cfg["vocab_size"], dtype=torch.float32, device=dev)
        laid = IcStepBatch()
        st = lib.ic_decoder_step(dec, ctypes.byref(hb), staging.data_ptr(), ints.data_ptr(), n, work.data_ptr(),
                                 work.numel(), lib_ws.data_ptr(), lib_ws.numel(), logits.data_ptr(),
                                 ctypes.byref(laid), stream)
        assert st == 0, lib.ic_decoder_last_error(dec).decode()
        torch.cuda.synchronize()
        assert lib.ic_decoder_workspace_bytes(dec, ctypes.byref(laid)) <= work.numel()
        return logits, laid

    got, laid = c_step([0, 1, 2], [prompts[0], prompts[1], prompts[2][:40]], [0, 0, 0], [[0, 149], [8], []])
    assert (laid.n_tokens, laid.n_requests, laid.n_want, laid.n_decode_rows) == (199, 3, 3, 0)
    want = ref.step([StepEntry("a", prompts[0], [0, 149]), StepEntry("b", prompts[1], [8]),
                     StepEntry("c", prompts[2][:40], [])])
    # the reference engine hands out pages in the same order, so even the cache slots agree; the logits must
    assert torch.equal(got, want)
    got, laid = c_step([1, 2, 0], [[5], prompts[2][40:], [7]], [9, 40, 150], [[0], [0, 29], [0]])
    assert (laid.n_decode_rows, laid.n_prefill_tiles, laid.want_rows_identity) == (2, 1, 0)
    want = ref.step([StepEntry("b", [5], [0]), StepEntry("c", prompts[2][40:], [0, 29]), StepEntry("a", [7], [0])])
    assert torch.equal(got, want)
    # a batch that does not add up is refused before anything is launched
    bad = IcHostBatch(5, 1, 0, 0, 0, 0, 0, 0, 0, 128, 0)
    assert lib.ic_decoder_step_ints(dec, ctypes.byref(bad)) == -1
