"""The step issued by native code: one call into the kernel library launches every kernel of a
step (csrc/decoder.hip behind csrc/infinicore_infer_engine.h), instead of one ctypes call per
kernel from the parts' Python ``forward``.  The reference's step function is native too
(src/models/jiuge/jiuge.cpp:114-298, called through include/infinicore_infer/models/jiuge.h:89-110).

It is a capability, not a requirement: a model takes this path when every part of it has a
native description (``Part.native_desc``); any other model is stepped by its parts' ``forward``
as before.  Both paths launch the same kernels with the same arguments, so their logits are
bit-equal (tested).
"""
import ctypes
from itertools import chain
from typing import Optional

import numpy as np
import torch

from ..kernels import ops
from ..kernels.lib import (MAX_CACHE_GROUPS, IcDecoderMeta, IcHostBatch, IcLayer, IcNorm, IcRunEntry, IcStepBatch,
                           KernelError, get_lib)


class NativeDecoder:
    """Owns the C-side decoder object of one engine's model and cache planes."""

    def __init__(self, handle, lib, vocab, keep):
        self._h = ctypes.c_void_p(handle)
        self._lib = lib
        self.vocab = vocab
        self._keep = keep                 # the description arrays and derived tensors the C side points into
        self._batch = IcStepBatch()
        self._batch_ref = ctypes.byref(self._batch)
        self._forward = lib.ic_decoder_forward
        self._bytes = lib.ic_decoder_workspace_bytes

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.ic_decoder_destroy(h)

    @classmethod
    def try_build(cls, engine) -> Optional["NativeDecoder"]:
        """A decoder for the engine's model, or None when some part has no native description."""
        model, rt = engine.model, engine.runtime
        if rt.attention_impl != "auto" or rt.gemm_impl != "auto" or len(engine.groups) > MAX_CACHE_GROUPS:
            return None
        emb, head = model.embedding.native_desc(), model.head.native_desc()
        fin = model.final_norm.native_desc()
        layers = [l.native_desc() for l in model.layers]
        if emb is None or head is None or not isinstance(fin, IcNorm) or not all(isinstance(l, IcLayer) for l in layers):
            return None
        if engine.has_state or any(g.planes != 2 for g in engine.groups) or \
                any(s not in engine._slot_group for s in range(model.spec.num_cache_slots())):
            return None                   # fixed-size state or a cache that is not keys and values: no built-in part has one
        scaled = model.head.deferred_norm(model.final_norm)
        if scaled is None:
            return None
        scaled_w = scaled.deferred()[0]
        lib = get_lib()
        # arrival counters of the prompt attention's cut walks: this engine's own, zero now and after every step
        counters = torch.zeros(ops.attention_prefill_counter_ints(), dtype=torch.int32, device=engine.device)
        layer_arr = (IcLayer * len(layers))(*layers)
        entries = []
        for e in model.schedule:
            k, v = engine.storage.kv(e.cache)
            entries.append(IcRunEntry(e.layer, int(e.writes_cache), engine._slot_group[e.cache], k.data_ptr(), v.data_ptr()))
        entry_arr = (IcRunEntry * len(entries))(*entries)
        meta = IcDecoderMeta(ops.dtype_code(rt.dtype), model.spec.hidden_size, model.spec.vocab_size, engine.page_size,
                             len(layers), len(entries), len(engine.groups), engine.cu_count, emb[1], head[1], emb[0],
                             head[0], fin, scaled_w.data_ptr(), counters.data_ptr())
        handle = lib.ic_decoder_create(ctypes.byref(meta), layer_arr, entry_arr)
        if not handle:
            raise KernelError("the native step function refused the model: %s"
                              % lib.ic_decoder_create_error().decode())
        return cls(handle, lib, model.spec.vocab_size, (layer_arr, entry_arr, meta, scaled_w, counters))

    def workspace_bytes_for_decode(self, n_requests: int) -> int:
        """Workspace bytes that any step of up to ``n_requests`` single tokens needs (with the most key
        splits the kernels take), for a workspace that recorded steps share and that must never grow."""
        b = IcStepBatch()
        b.n_tokens = b.n_requests = b.n_want = b.n_decode_rows = int(n_requests)
        b.want_rows_identity = b.decode_rows_identity = 1
        b.fixed_decode_splits = 64
        need = self._bytes(self._h, ctypes.byref(b))
        if need < 0:
            raise KernelError("native step: no workspace size for %d single tokens" % n_requests)
        return int(need)

    def step(self, engine, entries, starts):
        """A whole step from the entries themselves, the way the reference's inferBatch takes a batch
        (tokens, req_lens, req_pos, one cache per request; include/infinicore_infer/models/jiuge.h:89-110):
        native code lays the step's integers out in pinned memory, one copy takes them to the device,
        one call launches the kernels.  Returns float32 logits [wanted, vocab] or None."""
        lib, cache = self._lib, engine.cache
        R, ng = len(entries), len(engine.groups)
        lens = [len(e.tokens) for e in entries]
        T = sum(lens)
        tok = np.fromiter(chain.from_iterable(e.tokens for e in entries), dtype=np.int32, count=T)
        req_lens = np.array(lens, dtype=np.int32)
        req_pos = np.array(starts, dtype=np.int32)
        want_count = np.array([len(e.want) for e in entries], dtype=np.int32)
        n_want = int(want_count.sum())
        want = np.fromiter(chain.from_iterable(e.want for e in entries), dtype=np.int32, count=n_want)
        tables = [np.asarray(cache.block_table(e.req_id, g), dtype=np.int32) for g in range(ng) for e in entries]
        ptrs = (ctypes.c_void_p * (ng * R))(*[t.ctypes.data for t in tables])
        table_len = np.array([t.shape[0] for t in tables], dtype=np.int32)
        hb = IcHostBatch(T, R, tok.ctypes.data, req_lens.ctypes.data, req_pos.ctypes.data, want_count.ctypes.data,
                         want.ctypes.data, ctypes.cast(ptrs, ctypes.c_void_p), table_len.ctypes.data,
                         engine._tile_rows, 0)
        n = lib.ic_decoder_step_ints(self._h, ctypes.byref(hb))
        if n < 0:
            raise KernelError("native step: the batch is not valid (lengths, positions or block tables)")
        host = engine._ring.get(n)
        dev = engine._meta_dev
        if dev is None or dev.numel() < n:
            dev = engine._meta_dev = torch.empty(max(n, 4096), dtype=torch.int32, device=engine.device)
        b = self._batch
        st = lib.ic_decoder_pack(self._h, ctypes.byref(hb), host.data_ptr(), dev.data_ptr(), n, self._batch_ref)
        if st:
            raise KernelError("native step: laying out the batch failed (%d)" % st)
        dev[:n].copy_(host[:n], non_blocking=True)
        engine._ring.mark()
        return self._launch(engine.ws, "native")

    def _launch(self, workspace, workspace_name):
        """Launch the step that ``self._batch`` describes."""
        b = self._batch
        need = self._bytes(self._h, self._batch_ref)
        if need < 0:
            raise KernelError("native step: the batch description is not valid")
        ws = workspace.buffer(workspace_name, (need,), torch.uint8)
        logits = workspace.buffer("logits", (b.n_want, self.vocab), torch.float32) if b.n_want else None
        lib_ws = ops.library_workspace(ws.device)
        st = self._forward(self._h, self._batch_ref, ws.data_ptr(), need, lib_ws.data_ptr(), ops.MATMUL_WORKSPACE_BYTES,
                           logits.data_ptr() if logits is not None else None, ops.current_stream())
        if st:
            msg = self._lib.ic_decoder_last_error(self._h).decode()
            if st == -4:
                raise ops.NoLibraryAlgorithm("native step: " + msg)
            raise KernelError("native step: " + msg)
        return logits

    def forward(self, ctx, workspace_name: str = "native"):
        """Launch the step ``ctx`` describes; returns float32 logits [n_want, vocab] (a workspace view) or None."""
        b = self._batch
        b.n_tokens, b.n_requests, b.n_want = ctx.T, ctx.R, ctx.n_want
        b.n_decode_rows, b.n_prefill_tiles = ctx.n_decode_rows, ctx.n_prefill_tiles
        b.want_rows_identity, b.decode_rows_identity = int(ctx.want_rows_identity), int(ctx.decode_rows_identity)
        b.max_position, b.max_context = ctx.max_position, ctx.max_context
        b.fixed_decode_splits = ctx.fixed_decode_splits or 0
        b.tokens, b.positions, b.token_req = ctx.tokens.data_ptr(), ctx.positions.data_ptr(), ctx.token_req.data_ptr()
        b.want_rows = ctx.want_rows.data_ptr() if ctx.n_want else None
        b.decode_rows = ctx.decode_rows.data_ptr() if (ctx.decode_rows is not None and ctx.n_decode_rows) else None
        b.prefill_tiles = ctx.prefill_tiles.data_ptr() if ctx.n_prefill_tiles else None
        for g, (slots, tables) in enumerate(ctx.group_views):
            b.group_slots[g] = slots.data_ptr()
            b.group_tables[g] = tables.data_ptr()
            b.group_table_stride[g] = tables.stride(0)
        return self._launch(ctx.ws, workspace_name)
