"""Execution of the auto-batching graph on the HIP model: prefill per sequence, batched greedy decode.

Restates `tvm/llama_auto_batcher/llama_exec_graph.py:10-174`.  Differences that do not change results:
the argmax runs on the device and only the token ids cross to the host (the reference copies the full
fp32 logits and calls np.argmax, `:92,134-137`; ties resolve to the lowest index in both); prompts may be
given as token-id arrays when no tokenizer is configured; decode batches of a single adapter type run through the
native decode step and batches that mix adapter types through a graph-replayed per-operator step (bit-identical
tokens either way, see LlamaExecConfig.native_decode).
"""
from __future__ import annotations

import dataclasses
import os
import re

import numpy as np
import torch

from . import ops
from .exec_graph import ExecGraph


@dataclasses.dataclass
class LlamaExecConfig:
    max_prompt_len: int
    max_gen_len: int
    page_size: int
    # Run decode batches of one adapter type (or none) through the native decode step (one C call per step, graph
    # replay when several steps lie ahead) instead of one call per operator, and batches that mix adapter types
    # through the per-operator step recorded into a graph.  Same tokens: the native step with ids-based LoRA shrink
    # is bit-identical to the per-operator path.
    native_decode: bool = True
    # Let the native step compute the LoRA shrink of all adapters as extra rows of the base GEMV: the fastest form
    # while the adapters are few and low-rank, taken where it applies (every rank at most 16, one scaling, at most 64
    # sequences and no more adapters than twice the batch) and what the headline benchmark times.  It then also serves
    # batches that mix adapter types of one scaling, and rows without adapter, from the types' zero-padded union.
    # The fp32 summation order of x . A^T differs from the per-operator path, so a greedy token can differ from that
    # path at a near tie (against the oracle the two forms are equally close); False keeps the ids-based shrink, whose
    # tokens are bit-identical to the per-operator path.
    dense_lora: bool = True
    # Prefill the prompts of all requests in one forward pass instead of one pass per request (the reference's way).
    # Same arithmetic per token, but larger token counts take other GEMM kernels and summation orders, so the first
    # token of a request can differ from the per-request prefill at a near tie.
    batch_prefill: bool = False


class LlamaExecGraph(ExecGraph):
    def __init__(self, batchable_op_types=("decode",)):
        super().__init__(batchable_op_types)
        self.measure = False
        self.measure_file = None
        self.step_ms = []

    def set_exec_vars(self, vm, dev, params, tokenizer, seq_info, exec_config, eos_token_id=None, free_pages=None):
        self.vm = vm                  # a LlamaForCausalLM: entry points by name
        self.dev = dev
        self.params = params          # kept for signature parity; weights live inside `vm`
        self.tokenizer = tokenizer
        self.seq_info = seq_info
        self.exec_config = exec_config
        self.eos_token_id = eos_token_id if eos_token_id is not None else getattr(tokenizer, "eos_token_id", None)
        self.free_pages = free_pages
        self.measure = False
        self.kv_cache = None
        self.set_kv_cache(False)

    def set_kv_cache(self, delete_prev=True):
        if delete_prev:
            self.kv_cache = None
        n = self.seq_info.get_num_sequences()
        c = self.exec_config
        self.kv_cache = self.vm["create_paged_kv_cache"](
            n, n * (c.max_prompt_len + c.max_gen_len), c.max_prompt_len, c.page_size,
            free_pages=self.free_pages, max_seq_len=c.max_prompt_len + c.max_gen_len)

    def set_measuring(self, dest):
        """One millisecond value per line, one line per prefill and per decode step (`:48-50,70-74,116-132`)."""
        self.measure = True
        self.measure_file = open(dest if os.path.isabs(dest) else os.path.join(os.path.expanduser("~"), dest), "w")

    # ------------------------------------------------------------------ timing
    def _tic(self):
        if not self.measure:
            return None
        ev = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        torch.cuda.synchronize()
        ev[0].record()
        return ev

    def _toc(self, ev):
        if ev is None:
            return
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1])
        self.step_ms.append(ms)
        if self.measure_file is not None:
            self.measure_file.write(f"{ms}\n")
            self.measure_file.flush()                   # the file stays open across passes: keep it readable meanwhile

    # ------------------------------------------------------------------ operations
    def execute_encode_prompt(self, op):
        assert len(op.input_vars) == 1 and len(op.output_vars) == 1 and len(op.seqids) == 1, \
            "encode_prompt node must have exactly 1 input var, 1 output var and 1 seqid"
        prompt = op.input_vars[0].var
        if isinstance(prompt, str):
            assert self.tokenizer is not None, "a text prompt needs a tokenizer"
            ids = np.asarray(self.tokenizer(prompt)["input_ids"], dtype=np.int32).reshape(1, -1)
        else:
            ids = np.asarray(prompt, dtype=np.int32).reshape(1, -1)
        op.output_vars[0].var = ids

    def execute_prefill(self, op):
        if len(op.seqids) > 1:
            return self._prefill_batch(op)
        assert len(op.input_vars) == 1 and len(op.output_vars) == 1 and len(op.seqids) == 1, \
            "prefill node must have exactly 1 input var, 1 output var and 1 seqid"
        sid = op.seqids[0]
        tokens = op.input_vars[0].var
        self.kv_cache.add_sequence(sid)
        hidden = self.vm["embed"](torch.from_numpy(np.ascontiguousarray(tokens)))
        adapter = self.seq_info.get_adapter_info(sid)
        ev = self._tic()
        self.kv_cache.begin_forward([sid], [tokens.shape[1]])
        if adapter is None:
            logits, _ = self.vm["prefill_no_adapter"](hidden, self.kv_cache)
        else:
            logits, _ = self.vm[f"prefill_a{adapter['tid']}"](hidden, self.kv_cache, [adapter["wid"]])
        self.kv_cache.end_forward()
        self._toc(ev)
        op.output_vars[0].var = int(ops.argmax(logits).cpu()[0])

    def _prefill_batch(self, op):
        """The prompts of several requests in one forward pass (`LlamaExecConfig.batch_prefill`; the reference
        prefills one sequence per call, `:58-92`): the prompts are concatenated in request order, every token carries
        its request's adapter, attention stays inside each request's own pages, and the logits are taken at each
        prompt's last token."""
        n = len(op.seqids)
        assert len(op.input_vars) == n and len(op.output_vars) == n, "prefill node needs one input and one output var per sequence"
        prompts = [np.asarray(v.var, dtype=np.int32).reshape(-1) for v in op.input_vars]
        lens = [int(p.size) for p in prompts]
        T = sum(lens)
        per_type = {}                                           # adapter type -> weight id per token, -1 elsewhere
        start = 0
        for sid, L in zip(op.seqids, lens):
            self.kv_cache.add_sequence(sid)
            adapter = self.seq_info.get_adapter_info(sid)
            if adapter is not None:
                per_type.setdefault(adapter["tid"], np.full(T, -1, dtype=np.int32))[start:start + L] = adapter["wid"]
            start += L
        hidden = self.vm["embed"](torch.from_numpy(np.ascontiguousarray(np.concatenate(prompts))))
        ev = self._tic()
        self.kv_cache.begin_forward(list(op.seqids), lens)
        ids = self.vm._ids(T, {tid: (None, wids) for tid, wids in sorted(per_type.items())})
        logits = self.vm.forward(hidden, self.kv_cache, ids, self.vm._last_rows(self.kv_cache))
        self.kv_cache.end_forward()
        self._toc(ev)
        first = ops.argmax(logits).cpu().numpy()
        for i in range(n):
            op.output_vars[i].var = int(first[i])

    def check_seqs_finished(self, seqs_2_decode, outputs):
        return [sid for sid in seqs_2_decode
                if outputs[sid][-1] != self.eos_token_id and len(outputs[sid]) < self.seq_info.get_max_gen_len(sid)]

    def execute_decode(self, op):
        assert len(op.input_vars) == len(op.output_vars), "decode node needs as many output vars as input vars"
        assert len(op.input_vars) == len(op.seqids), "decode node needs one sequence id per input var"
        seqs, original_positions = self.seq_info.order_seqs(op.seqids)
        outputs = {sid: [int(op.input_vars[original_positions[i]].var)] for i, sid in enumerate(seqs)}
        ordered = list(seqs)
        # As in the reference (`:102-141`), the finish rule (`:94-100`) is applied only after a decode step: every
        # sequence takes at least one step after its prefill, also when its first token is EOS or max_gen_len is 1.
        while seqs:
            method, params = self.seq_info.get_decode_method(seqs)
            if getattr(self.exec_config, "native_decode", False):
                dense = len(seqs) <= 64 and self._dense_ok(method)       # the dense shrink serves at most 64 sequences
                seqs = self._decode_native(seqs, outputs, method, params, dense) if dense or not method.startswith("mixed_decode") \
                    else self._decode_session(seqs, outputs, method, params)
                continue
            tokens = torch.tensor([outputs[sid][-1] for sid in seqs], dtype=torch.int32)
            hidden = self.vm["embed"](tokens)
            ev = self._tic()
            self.kv_cache.begin_forward(seqs, [1] * len(seqs))
            logits, _ = self.vm[method](hidden, self.kv_cache, *params)
            self.kv_cache.end_forward()
            self._toc(ev)
            nxt = ops.argmax(logits).cpu().numpy()
            for i, sid in enumerate(seqs):
                outputs[sid].append(int(nxt[i]))
            seqs = self.check_seqs_finished(seqs, outputs)
        for i, sid in enumerate(ordered):
            op.output_vars[original_positions[i]].var = np.asarray(outputs[sid], dtype=np.int64)

    def _decode_native(self, seqs, outputs, method, params, dense=False):
        """Decode this batch with the native step until its composition changes (a sequence reaches its length
        limit or emits EOS); returns the sequences still running.  Without an EOS id the number of steps until
        the next length limit is known in advance and the tokens come back in one copy."""
        from .decode_session import NativeDecodeSession
        if method.startswith("mixed_decode"):
            # several types, or one type beside rows without adapter: rows of the types' padded union, -1 = no adapter
            tids = self._method_tids(method)
            pairs = {t: (params[2 * i], params[2 * i + 1]) for i, t in enumerate(tids)}
            tid = tuple(tids)
            wids = self.vm.union_rows(tids, len(seqs), pairs)
        else:
            tid = int(method[len("decode_a"):]) if method != "decode_no_adapter" else 0
            wids = params[0] if params else None
        last = [outputs[sid][-1] for sid in seqs]
        ahead = max(1, min(self.seq_info.get_max_gen_len(sid) - len(outputs[sid]) for sid in seqs))
        sess = NativeDecodeSession(self.vm, self.kv_cache, seqs, wids, last, tid=tid, use_graph=ahead >= 8, dense_lora=None if dense else False)
        if self.eos_token_id is None and not self.measure:
            for _ in range(ahead):
                sess.step(keep_history=True)
            toks = torch.stack(sess.history).cpu().numpy()             # [ahead, batch]
            for i, sid in enumerate(seqs):
                outputs[sid].extend(int(t) for t in toks[:, i])
            return self.check_seqs_finished(seqs, outputs)
        while True:
            ev = self._tic()
            nxt = sess.step()
            self._toc(ev)
            nxt = nxt.cpu().numpy()
            for i, sid in enumerate(seqs):
                outputs[sid].append(int(nxt[i]))
            left = self.check_seqs_finished(seqs, outputs)
            if len(left) != len(seqs):
                return left

    @staticmethod
    def _method_tids(method):
        return [int(t) for t in re.findall(r"_a(\d+)", method)]

    def _dense_ok(self, method):
        """Whether the native step with the dense shrink serves this entry point: asked for in the configuration,
        ranks at most 16, and one scaling over its adapter types (they are served from their padded union)."""
        types = [self.vm.lora_types[t] for t in self._method_tids(method)]
        return bool(getattr(self.exec_config, "dense_lora", False) and types and max(lt.r for lt in types) <= 16
                    and len({lt.scaling for lt in types}) == 1)

    def _decode_session(self, seqs, outputs, method, params):
        """A batch that mixes adapter types (`mixed_decode_a{i}_a{j}...`): the per-operator step with the tokens,
        positions and context lengths kept on the device, replayed from a graph when enough steps lie ahead.  Same
        kernels in the same order as the call-per-step path, so the same tokens."""
        from .decode_session import DecodeSession
        tids = self._method_tids(method)
        pairs = {tid: (params[2 * i], params[2 * i + 1]) for i, tid in enumerate(tids)}
        last = [outputs[sid][-1] for sid in seqs]
        ahead = max(1, min(self.seq_info.get_max_gen_len(sid) - len(outputs[sid]) for sid in seqs))
        sess = DecodeSession(self.vm, self.kv_cache, seqs, self.vm._ids(len(seqs), pairs), last, use_graph=ahead >= 8)
        if self.eos_token_id is None and not self.measure:
            for _ in range(ahead):
                sess.step(keep_history=True)
            toks = torch.stack(sess.history).cpu().numpy()             # [ahead, batch]
            for i, sid in enumerate(seqs):
                outputs[sid].extend(int(t) for t in toks[:, i])
            return self.check_seqs_finished(seqs, outputs)
        while True:
            ev = self._tic()
            nxt = sess.step()
            self._toc(ev)
            nxt = nxt.cpu().numpy()
            for i, sid in enumerate(seqs):
                outputs[sid].append(int(nxt[i]))
            left = self.check_seqs_finished(seqs, outputs)
            if len(left) != len(seqs):
                return left

    def execute_decode_answer(self, op):
        assert len(op.input_vars) == 1 and len(op.output_vars) == 1 and len(op.seqids) == 1, \
            "decode_answer node must have exactly 1 input var, 1 output var and 1 seqid"
        ids = op.input_vars[0].var
        op.output_vars[0].var = self.tokenizer.decode(ids) if self.tokenizer is not None else ids

    def execute_print(self, op):
        if self.measure:
            return
        assert len(op.input_vars) == 1 and len(op.seqids) == 1, "print node must have exactly 1 input var and 1 seqid"
        print(f"Answer for Sequence {op.seqids[0]} {op.input_vars[0].var}")

    def execute_op(self, op):
        fn = {"encode_prompt": self.execute_encode_prompt, "prefill": self.execute_prefill,
              "decode": self.execute_decode, "decode_answer": self.execute_decode_answer,
              "print": self.execute_print}.get(op.op_type)
        if fn is None:
            print(f"[ERROR] unknown op_type: {op.op_type}")
            return
        fn(op)
