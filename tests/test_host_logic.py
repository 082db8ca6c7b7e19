"""Integer host logic (no GPU): sequence info, decode-method selection, graph fusion, page bookkeeping,
synthetic-input determinism.  Expected values are worked out by hand from the reference's request mix
(`tvm/llama_auto_batcher/user_example.py:7-39`)."""
import numpy as np
import pytest
import torch

from conftest import load_pkg


def _user_example_seq_info():
    si = load_pkg("seq_info").LlamaSeqInfo(32)
    L = load_pkg("lora").LoraConfig
    mix = [None, (L(64, 32), 0), (L(64, 32), 0), (L(64, 32), 1), (L(64, 32), 2), (L(32, 16), 0), (L(32, 16), 1)]
    for sid, m in enumerate(mix):
        si.add_sequence(sid)
        if m is not None:
            si.set_adapter(sid, m[0], m[1])
    return si


def test_seq_info_user_example():
    si = _user_example_seq_info()
    assert [c.r for c in si.get_adapter_configs()] == [64, 32]
    assert si.get_num_adapters_per_type() == [3, 2] and si.get_wids_per_type() == [{0, 1, 2}, {0, 1}]
    sids = list(range(7))
    ordered, pos = si.order_seqs(sids)
    assert ordered == [0, 1, 2, 3, 4, 5, 6] and pos == [0, 1, 2, 3, 4, 5, 6]
    name, params = si.get_decode_method(ordered)
    assert name == "mixed_decode_a0_a1"
    assert params == [[1, 2, 3, 4], [0, 0, 1, 2], [5, 6], [0, 1]]
    assert si.get_decode_method([1, 2, 3, 4]) == ("decode_a0", [[0, 0, 1, 2]])
    assert si.get_decode_method([0]) == ("decode_no_adapter", [])
    assert si.get_decode_method([5, 1]) == ("mixed_decode_a0_a1", [[1], [0], [0], [0]])
    assert si.get_decode_method([0, 6]) == ("mixed_decode_a1", [[1], [1]])


def test_order_seqs_is_stable_and_puts_no_adapter_first():
    si = _user_example_seq_info()
    ordered, pos = si.order_seqs([6, 4, 0, 2, 5, 1, 3])
    assert ordered == [0, 2, 1, 3, 4, 5, 6]               # (has adapter, tid, wid); ties keep input order
    assert pos == [2, 3, 5, 6, 1, 4, 0]
    si2 = load_pkg("seq_info").LlamaSeqInfo(8)
    si2.add_sequence(3)
    si2.add_sequence(1)
    assert si2.order_seqs([3, 1]) == ([3, 1], [0, 1])      # no adapter types: identity


def test_seq_info_max_gen_len_and_duplicates(capsys):
    si = load_pkg("seq_info").LlamaSeqInfo(10)
    si.add_sequence(0)
    with pytest.raises(AssertionError):
        si.add_sequence(0)
    si.set_max_gen_len(0, 50)
    assert si.get_max_gen_len(0) == 10 and "[WARN]" in capsys.readouterr().out
    si.set_max_gen_len(0, None)
    assert si.get_max_gen_len(0) == 10


def test_exec_graph_fusion_levels():
    """Seven requests: after fusion there is one decode node holding all seven sequences; the other
    levels keep one node per request (exec_graph.py:85-107)."""
    ab = load_pkg("auto_batcher").LlamaAutoBatcherClass()
    L = load_pkg("lora").LoraConfig
    for i in range(7):
        v = ab.create_var(np.arange(4))
        if i:
            ab.set_adapter(L(64, 32) if i < 5 else L(32, 16), wid=i % 3)
        r = ab.generate(v, max_gen_len=10 + i)
        ab.print(r)
    g = ab.graph
    assert g.get_max_batch_sizes() == {"decode": 1}
    g.fuse_batchable_ops()
    assert g.get_max_batch_sizes() == {"decode": 7}
    ops_levels = [[n.op_type for n in lvl] for lvl in g.levels() if lvl and hasattr(lvl[0], "op_type")]
    assert ops_levels == [["encode_prompt"] * 7, ["prefill"] * 7, ["decode"], ["decode_answer"] * 7, ["print"] * 7]
    dec = [n for lvl in g.levels() for n in lvl if getattr(n, "op_type", None) == "decode"][0]
    assert dec.seqids == list(range(7)) and len(dec.input_vars) == 7 and len(dec.output_vars) == 7
    assert ab.seq_info.get_max_gen_len(3) == 13
    assert all(v.ops == [dec] for v in dec.input_vars)


def test_exec_graph_fuses_prefill_too_when_it_is_batchable():
    """With "prefill" among the batchable operation types (what `LlamaExecConfig.batch_prefill` asks compile() for),
    the prefills of all requests fold into one operation whose variables and sequence ids stay aligned, and the
    decode fusion after it is unchanged."""
    ab = load_pkg("auto_batcher").LlamaAutoBatcherClass()
    outs = [ab.generate(ab.create_var(np.arange(3 + i)), max_gen_len=4) for i in range(5)]
    g = ab.graph
    g.batchable_op_types += ("prefill",)
    g.fuse_batchable_ops()
    assert g.get_max_batch_sizes() == {"prefill": 5, "decode": 5}
    ops_levels = [[n.op_type for n in lvl] for lvl in g.levels() if lvl and hasattr(lvl[0], "op_type")]
    assert ops_levels == [["encode_prompt"] * 5, ["prefill"], ["decode"], ["decode_answer"] * 5]
    pre = next(n for n in g.op_nodes if n.op_type == "prefill")
    dec = next(n for n in g.op_nodes if n.op_type == "decode")
    assert pre.seqids == dec.seqids == list(range(5))
    assert [v.id for v in pre.output_vars] == [v.id for v in dec.input_vars]
    assert [v.ops[0].output_vars[0] for v in dec.output_vars] == outs


def test_exec_graph_unfused_keeps_separate_decodes():
    ab = load_pkg("auto_batcher").LlamaAutoBatcherClass()
    for _ in range(3):
        ab.generate(ab.create_var(np.arange(3)), max_gen_len=4)
    kinds = [n.op_type for lvl in ab.graph.levels() for n in lvl if hasattr(n, "op_type")]
    assert kinds.count("decode") == 3


def test_synth_is_deterministic_and_device_independent_logic():
    synth = load_pkg("synth")
    a = synth.normal(5, "x", (1000,), 0.02, torch.float16)
    b = synth.normal(5, "x", (1000,), 0.02, torch.float16)
    c = synth.normal(6, "x", (1000,), 0.02, torch.float16)
    assert torch.equal(a, b) and not torch.equal(a, c)
    big = synth.normal(5, "y", (200000,), 1.0, torch.float32).numpy()
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1.0) < 0.01 and np.abs(big).max() < 3.47
    u = synth.uniform(5, "u", (100000,), 0.5, torch.float32).numpy()
    assert u.min() >= -0.5 and u.max() <= 0.5 and abs(u.std() - 0.5 / np.sqrt(3)) < 0.01
    r = synth.randint(5, "r", (100000,), 32000).numpy()
    assert r.min() >= 0 and r.max() < 32000 and len(np.unique(r)) > 30000 * 0.9
    p = synth.permutation(5, "p", 1000)
    assert sorted(p.tolist()) == list(range(1000))
    # the hash is pure integer arithmetic: known answers guard against silent changes of the generator
    assert synth.hash32(0, "kat", 4).tolist() == synth.hash32(0, "kat", 6).tolist()[:4]
    assert synth.hash32(0, "kat", 3, offset=2).tolist() == synth.hash32(0, "kat", 5).tolist()[2:]


def test_workload_configs():
    synth = load_pkg("synth")
    c3 = synth.config3()
    assert c3.adapter_ids.tolist() == [i % 16 for i in range(32)] and c3.shape.intermediate_size == 11008
    c5 = synth.config5()
    assert c5.ctx_lens.min() >= 128 and c5.ctx_lens.max() <= 2048 and len(c5.adapter_ids) == 256
    counts = np.bincount(c5.adapter_ids, minlength=256)
    assert counts[0] == counts.max() and counts[0] > 20          # Zipf: adapter 0 is the most popular
    c4 = synth.config4()
    assert c4.lora.r == 64 and len(c4.lora.targets) == 7


def test_adapter_files_round_trip_and_wid_translation(tmp_path):
    """Adapters written in the reference's file layout (`r{rank}_a{wid}.safetensors`, PEFT-oriented fp32 tensors) load
    into stacked tables; weight ids that are not 0..n-1 in order are translated to table rows (the reference indexes
    the stack with the raw id, `compile_tvm.py:298-313` vs `llama_exec_graph.py:83`)."""
    import torch
    from safetensors.torch import load_file
    synth, af = load_pkg("synth"), load_pkg("adapter_files")
    shape = synth.LlamaShape(hidden_size=64, intermediate_size=96, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=2, head_dim=16, vocab_size=50)
    d = str(tmp_path / "lora_adapters")
    af.write_synthetic_adapters(d, shape, ranks=(8, 16), n_adapters=5, targets=("q_proj", "v_proj"), seed=3)
    f = load_file(af.adapter_path(d, 16, 4))
    assert sorted(f) == sorted(f"layers.{l}.self_attn.{p}.lora_{w}.weight" for l in range(2) for p in ("q_proj", "v_proj") for w in "AB")
    assert f["layers.1.self_attn.v_proj.lora_B.weight"].shape == (32, 16) and f["layers.0.self_attn.q_proj.lora_A.weight"].dtype == torch.float32
    lt = af.load_lora_type(d, 16, 8.0, [4, 0, 2], shape, device="cpu")
    assert lt.n_adapters == 3 and lt.scaling == 0.5 and lt.row_of == {4: 0, 0: 1, 2: 2}
    A, B = lt.tables[(1, "v_proj")]
    assert A.shape == (3, 16, 64) and B.shape == (3, 32, 16) and A.dtype == torch.float16
    want = load_file(af.adapter_path(d, 16, 2))["layers.1.self_attn.v_proj.lora_A.weight"].half()
    assert torch.equal(A[2], want)
    assert list(lt.rows(np.array([2, -1, 4, 0], dtype=np.int32))) == [2, -1, 0, 1]
    with pytest.raises(ValueError):
        lt.rows(np.array([3], dtype=np.int32))
    with pytest.raises(FileNotFoundError):
        af.load_lora_type(d, 16, 8.0, [7], shape, device="cpu")
    with pytest.raises(ValueError):
        af.load_lora_type(d, 16, 8.0, [1, 1], shape, device="cpu")


class _StubTokenizer:
    """The three things the front end asks of a tokenizer (`tvm/llama_auto_batcher/llama_exec_graph.py:52-56,143-147`,
    `llama_auto_batcher.py:21`): call -> {'input_ids': ...}, decode, eos_token_id.  One token per character."""
    eos_token_id = 3

    def __call__(self, text, **kwargs):
        ids = [ord(c) - 28 for c in text]
        return {"input_ids": [ids] if kwargs.get("return_tensors") else ids}

    def decode(self, ids):
        return "".join(chr(int(i) + 28) for i in np.asarray(ids).reshape(-1))


def test_text_prompt_path_with_a_stub_tokenizer():
    """encode_prompt turns a text prompt into a [1, n] int32 id array through the tokenizer (id arrays pass through
    unchanged), decode_answer turns generated ids back into text, the EOS id defaults to the tokenizer's; both node
    kinds insist on exactly one input, one output and one sequence, as the reference's asserts do."""
    eg, xg = load_pkg("llama_exec_graph"), load_pkg("exec_graph")
    g = eg.LlamaExecGraph()
    g.tokenizer = _StubTokenizer()
    text = "hello auto-batching"
    v_in, v_ids, v_out, v_txt = (xg.VarNode(i, None) for i in range(4))
    v_in.var = text
    enc = xg.OpNode("encode_prompt", [v_in], [v_ids], [0])
    g.execute_op(enc)
    assert v_ids.var.dtype == np.int32 and v_ids.var.shape == (1, len(text))
    assert v_ids.var.reshape(-1).tolist() == [ord(c) - 28 for c in text]
    v_in.var = np.array([5, 6, 7])                                    # token ids instead of text: no tokenizer call
    g.execute_op(enc)
    assert v_ids.var.tolist() == [[5, 6, 7]] and v_ids.var.dtype == np.int32
    v_out.var = np.array([76, 77, 78], np.int32)
    dec = xg.OpNode("decode_answer", [v_out], [v_txt], [0])
    g.execute_op(dec)
    assert v_txt.var == "hij"
    g.tokenizer = None                                                # without a tokenizer the ids are the answer ...
    g.execute_op(dec)
    assert v_txt.var is v_out.var
    v_in.var = "text"                                                 # ... and a text prompt is refused
    with pytest.raises(AssertionError):
        g.execute_op(enc)
    with pytest.raises(AssertionError):
        g.execute_op(xg.OpNode("encode_prompt", [v_in, v_in], [v_ids], [0]))
    with pytest.raises(AssertionError):
        g.execute_op(xg.OpNode("decode_answer", [v_out], [v_txt], [0, 1]))
    # the EOS id is the tokenizer's unless one is given (set_exec_vars reads it before it builds the cache)
    class _NoCacheGraph(eg.LlamaExecGraph):
        def set_kv_cache(self, delete_prev=True):
            pass
    g2 = _NoCacheGraph()
    g2.set_exec_vars(None, "cpu", None, _StubTokenizer(), None, None)
    assert g2.eos_token_id == 3
    g2.set_exec_vars(None, "cpu", None, _StubTokenizer(), None, None, eos_token_id=11)
    assert g2.eos_token_id == 11
