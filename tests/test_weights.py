"""Weights: safetensors reading and writing, loading by name, the one error that lists
everything that does not fit, dtypes, the tied head, random-weights mode."""
import json
import os
import struct

import pytest
import torch

import tiny_models as TM
from infernum_amd.config import model_spec_for
from infernum_amd.models import DecoderModel
from infernum_amd.parts import Runtime
from infernum_amd.weights import (SafetensorsError, WeightError, load_weights, open_model_tensors, random_tensors,
                                  write_random_model, write_safetensors)

CPU = torch.device("cpu")


def _model(name, dtype):
    return DecoderModel(model_spec_for(TM.tiny_config(name), **TM.SPEC_KW[name]), Runtime(CPU, dtype))


def _rewrite(model_dir, change):
    """Read all tensors of a folder, let ``change`` edit the dict, write them back."""
    path = os.path.join(model_dir, "model.safetensors")
    tensors = {n: e.read().clone() for n, e in open_model_tensors(model_dir).items()}
    change(tensors)
    write_safetensors(path, tensors.items())


def test_safetensors_round_trip(tmp_path):
    ts = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int64).reshape(2, 3),
          "d": torch.randn(2, 2, 2).to(torch.float16), "e": torch.empty(0, 4)}
    write_safetensors(str(tmp_path / "model.safetensors"), ts.items())
    got = open_model_tensors(str(tmp_path))
    assert sorted(got) == sorted(ts)
    for n, t in ts.items():
        assert got[n].dtype == t.dtype and tuple(got[n].shape) == tuple(t.shape)
        assert torch.equal(got[n].read(), t)
    # the layout is the published one: u64 length, JSON, bytes
    raw = (tmp_path / "model.safetensors").read_bytes()
    (n,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + n])
    assert header["a"]["dtype"] == "F32" and header["a"]["shape"] == [3, 5]
    b, e = header["a"]["data_offsets"]
    assert raw[8 + n + b:8 + n + e] == ts["a"].numpy().tobytes()


def test_safetensors_errors(tmp_path):
    with pytest.raises(SafetensorsError, match="No .safetensors files found"):
        open_model_tensors(str(tmp_path))
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="shorter"):
        open_model_tensors(str(tmp_path))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        open_model_tensors(str(tmp_path))
    p.write_bytes(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(SafetensorsError, match="not JSON"):
        open_model_tensors(str(tmp_path))
    h = json.dumps({"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(h)) + h + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="offsets"):
        open_model_tensors(str(tmp_path))
    h = json.dumps({"x": {"dtype": "Q4", "shape": [4], "data_offsets": [0, 2]}}).encode()
    p.write_bytes(struct.pack("<Q", len(h)) + h + b"\0" * 2)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        open_model_tensors(str(tmp_path))


def test_tensor_in_two_files_is_refused(tmp_path):
    write_safetensors(str(tmp_path / "a.safetensors"), [("w", torch.zeros(2))])
    write_safetensors(str(tmp_path / "b.safetensors"), [("w", torch.zeros(2))])
    with pytest.raises(SafetensorsError, match="both"):
        open_model_tensors(str(tmp_path))


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_random_model_loads_and_names_are_the_architectures(tmp_path, name):
    d = TM.write_tiny(name, str(tmp_path), dtype=torch.float32)
    cfg = TM.tiny_config(name)
    names = set(open_model_tensors(d))
    # infernum-llama/src/graph_builder.rs:201-364
    want = {"model.embed_tokens.weight", "model.norm.weight"}
    for i in range(cfg.num_hidden_layers):
        for t in ("input_layernorm", "post_attention_layernorm", "self_attn.q_proj", "self_attn.k_proj",
                  "self_attn.v_proj", "self_attn.o_proj", "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"):
            want.add(f"model.layers.{i}.{t}.weight")
    if not cfg.tie_word_embeddings:
        want.add("lm_head.weight")
    assert names == want
    m = _model(name, torch.float32)
    load_weights(m, d)
    assert m.embedding.table.dtype == torch.float32
    if cfg.tie_word_embeddings:
        assert m.head.weight.data_ptr() == m.embedding.table.data_ptr()      # one buffer, no copy
    else:
        assert m.head.weight.data_ptr() != m.embedding.table.data_ptr()


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = TM.write_tiny("B", str(tmp_path), dtype=torch.float32)

    def change(t):
        del t["model.layers.1.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.7.extra.weight"] = torch.zeros(3)
        t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 128)      # should be [32, 128]
        t["model.layers.2.input_layernorm.weight"] = torch.zeros(127)
    _rewrite(d, change)
    with pytest.raises(WeightError) as e:
        load_weights(_model("B", torch.float32), d)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert len(err.wrong_shape) == 2
    msg = str(err)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (2)", "model.layers.7.extra.weight",
                   "model.layers.0.self_attn.k_proj.weight: expected [32, 128] got [64, 128]",
                   "model.layers.2.input_layernorm.weight: expected [128] got [127]"):
        assert needle in msg, needle


def test_head_falls_back_to_the_embedding_by_file_contents(tmp_path):
    # infernum-cuda/src/inner/cuda_graph_engine.rs:225-232: by what the file holds, not by tie_word_embeddings
    d = TM.write_tiny("B", str(tmp_path), dtype=torch.float32)       # B says untied
    _rewrite(d, lambda t: t.pop("lm_head.weight"))
    m = _model("B", torch.float32)
    load_weights(m, d)
    assert m.head.weight.data_ptr() == m.embedding.table.data_ptr()
    # and a tied configuration whose file does hold a head uses that head
    d2 = TM.write_tiny("A", str(tmp_path / "a"), dtype=torch.float32)
    head = torch.randn(256, 64)
    _rewrite(d2, lambda t: t.__setitem__("lm_head.weight", head))
    m2 = _model("A", torch.float32)
    load_weights(m2, d2)
    assert torch.equal(m2.head.weight, head)


def test_dtypes_matrices_follow_compute_dtype_32bit_tensors_stay(tmp_path):
    d = TM.write_tiny("B", str(tmp_path), dtype=torch.bfloat16)

    def change(t):
        t["model.norm.weight"] = t["model.norm.weight"].to(torch.float32) + 1e-4    # not a bf16 value
    _rewrite(d, change)
    m = _model("B", torch.bfloat16)
    load_weights(m, d)
    assert m.embedding.table.dtype == torch.bfloat16 and m.blocks[0].mixer.w_qkv.dtype == torch.bfloat16
    assert m.final_norm.weight.dtype == torch.float32                       # stored in 32-bit: stays so
    assert (m.final_norm.weight != m.final_norm.weight.to(torch.bfloat16).float()).any()
    assert m.blocks[0].mixer_norm.weight.dtype == torch.bfloat16            # stored in bf16: stays bf16
    m32 = _model("B", torch.float32)
    load_weights(m32, d)                                                    # 32-bit path: everything widened
    assert m32.embedding.table.dtype == torch.float32 and m32.blocks[0].mixer_norm.weight.dtype == torch.float32
    assert torch.equal(m32.embedding.table, m.embedding.table.float())


def test_integer_tables_become_int32():
    from infernum_amd.parts import WeightSpec
    from infernum_amd.weights.loader import _convert
    t = _convert(torch.arange(5, dtype=torch.int64), WeightSpec((5,), follows_compute_dtype=False), Runtime(CPU, torch.bfloat16))
    assert t.dtype == torch.int32 and t.tolist() == [0, 1, 2, 3, 4]


def test_fused_matrices_are_the_row_concatenation(tmp_path):
    d = TM.write_tiny("A", str(tmp_path), dtype=torch.float32)
    raw = {n: e.read() for n, e in open_model_tensors(d).items()}
    m = _model("A", torch.float32)
    load_weights(m, d)
    p = "model.layers.1."
    want = torch.cat([raw[p + "self_attn.q_proj.weight"], raw[p + "self_attn.k_proj.weight"],
                      raw[p + "self_attn.v_proj.weight"]])
    assert torch.equal(m.blocks[1].mixer.w_qkv, want)
    assert torch.equal(m.blocks[1].feed_forward.w_gate_up, torch.cat([raw[p + "mlp.gate_proj.weight"],
                                                                       raw[p + "mlp.up_proj.weight"]]))


def test_random_weights_depend_on_seed_and_name_only(tmp_path):
    cfg = TM.tiny_config("B")
    a = dict(random_tensors(cfg, 1, torch.float32, **TM.SPEC_KW["B"]))
    b = dict(random_tensors(cfg, 1, torch.float32, **TM.SPEC_KW["B"]))
    c = dict(random_tensors(cfg, 2, torch.float32, **TM.SPEC_KW["B"]))
    assert all(torch.equal(a[n], b[n]) for n in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    # a model with fewer layers draws the same values for the tensors it shares
    small = dict(random_tensors(cfg.replace(num_hidden_layers=1), 1, torch.float32, **TM.SPEC_KW["B"]))
    assert all(torch.equal(small[n], a[n]) for n in small)
    # distributions: N(0, 0.02) matrices, U(0.5, 1.5) norms
    w = a["model.layers.0.mlp.gate_proj.weight"]
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    n = a["model.layers.0.input_layernorm.weight"]
    assert 0.5 <= n.min().item() and n.max().item() <= 1.5 and n.std().item() > 0.1
    ones = dict(random_tensors(TM.tiny_config("A"), 0, torch.float32))["model.norm.weight"]
    assert torch.equal(ones, torch.ones(64))


def test_write_random_model_writes_a_folder_that_reads_back(tmp_path):
    cfg = TM.tiny_config("C")
    d = write_random_model(cfg, str(tmp_path / "m"), 5, dtype=torch.bfloat16)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    from infernum_amd.config import load_config
    assert load_config(d) == cfg
    assert all(e.dtype == torch.bfloat16 for e in open_model_tensors(d).values())


def test_random_values_are_a_function_of_the_element_alone(monkeypatch):
    """The same numbers whether a tensor is made in one piece or in several, and a normal distribution."""
    from infernum_amd.parts.base import WeightSpec
    from infernum_amd.weights import random_init as R
    spec = WeightSpec((37, 1001), ("normal", 0.5))
    whole = R.draw(spec, 3, "w", torch.device("cpu"))
    monkeypatch.setattr(R, "_CHUNK", 1000)
    assert torch.equal(R.draw(spec, 3, "w", torch.device("cpu")), whole)
    assert not torch.equal(R.draw(spec, 3, "v", torch.device("cpu")), whole)
    z = R.draw(WeightSpec((1 << 20,), ("normal", 1.0)), 0, "z", torch.device("cpu")).double()
    assert abs(z.mean().item()) < 5e-3 and abs(z.var().item() - 1) < 5e-3
    assert abs((z ** 3).mean().item()) < 2e-2 and abs((z ** 4).mean().item() - 3) < 5e-2
    assert abs((z[1:] * z[:-1]).mean().item()) < 5e-3            # neighbours are not correlated
    assert 4.0 < z.abs().max().item() < 5.0
    u = R.draw(WeightSpec((1 << 16,), ("uniform", -1.0, 3.0)), 0, "u", torch.device("cpu")).double()
    assert -1.0 <= u.min().item() < -0.99 and 2.99 < u.max().item() < 3.0 and abs(u.mean().item() - 1.0) < 2e-2


def test_tensors_come_part_by_part_and_a_shared_one_is_made_once(tmp_path):
    """Loading asks for a part's tensors when that part is loaded and keeps none that the part did not keep, so the
    originals of a fused matrix are gone before the next part's come; a tied head's tensor is made once."""
    import weakref
    from infernum_amd.weights.loader import LazyTensors
    made = []
    lazy = LazyTensors({"a": "k", "b": "k", "c": "c"}, lambda name, key: made.append((name, key)) or torch.zeros(3))
    a = lazy["a"]
    assert lazy["b"] is a and made == [("a", "k")] and "c" in lazy and "d" not in lazy
    ref = weakref.ref(lazy["c"])
    assert ref() is None and made == [("a", "k"), ("c", "c")]         # nothing but the caller held it
    assert not lazy._kept                                              # the shared one was let go with its last name
    # through the model: when a block's fused matrix is built, no tensor of an earlier block is alive any more
    m = _model("A", torch.float32)
    alive = []
    expected = m.expected_weights()
    keys = {n: n for n in expected}

    def make(name, key):
        assert not [r for r in alive if r[1]() is not None and r[0].split(".")[:3] != name.split(".")[:3]
                    and "q_proj" in r[0]], name
        t = torch.zeros(expected[name].shape)
        alive.append((name, weakref.ref(t)))
        return t

    m.load_weights(LazyTensors(keys, make))
    assert len(alive) == len(expected)
    # the tied configuration on random weights: head and embedding are one buffer
    from infernum_amd.weights.random_init import random_weights_on_device
    random_weights_on_device(m, 3)
    assert m.head.weight.data_ptr() == m.embedding.table.data_ptr()
