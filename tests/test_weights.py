"""Safetensors container, name-driven loading with one complete error, random-weights mode (no GPU)."""
import json
import os

import pytest
import torch

from rustinfer_amd.config import LlamaConfig
from rustinfer_amd.models.llama import build_llama
from rustinfer_amd.weights import (SafetensorsReader, WeightError, check_checkpoint, random_tensors,
                                   write_random_model, write_safetensors)
from helpers import TINY


def cfg_of(name):
    return LlamaConfig.from_dict(TINY[name][0])


def test_container_round_trip_and_library_agrees(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
         "c": torch.arange(6, dtype=torch.int32).reshape(2, 3), "d": torch.zeros(0, 4)}
    p = str(tmp_path / "model.safetensors")
    write_safetensors(p, t, metadata={"k": "v"})
    r = SafetensorsReader(str(tmp_path))
    assert sorted(r.names()) == ["a", "b", "c", "d"]
    for k, v in t.items():
        got = r.tensor(k)
        assert got.dtype == v.dtype and got.shape == v.shape and torch.equal(got, v)
    from safetensors.torch import load_file            # an independent reader of the same bytes
    lib = load_file(p)
    assert all(torch.equal(lib[k], v) for k, v in t.items())


def test_sharded_folder(tmp_path):
    write_safetensors(str(tmp_path / "s1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(str(tmp_path / "s2.safetensors"), {"b": torch.zeros(3)})
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    r = SafetensorsReader(str(tmp_path))
    assert torch.equal(r.tensor("a"), torch.ones(2)) and torch.equal(r.tensor("b"), torch.zeros(3))


def test_the_folder_is_searched_as_the_reference_searches_it(tmp_path):
    """An index of any prefix comes first, then model.safetensors, then a lone .safetensors file
    (safetensors.rs:62-101)."""
    d = tmp_path / "lone"
    d.mkdir()
    write_safetensors(str(d / "weights.safetensors"), {"a": torch.ones(2)})
    assert SafetensorsReader(str(d)).names() == ["a"]
    write_safetensors(str(d / "other.safetensors"), {"b": torch.ones(2)})
    with pytest.raises(WeightError, match="several .safetensors files"):
        SafetensorsReader(str(d))
    (d / "net.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"a": "weights.safetensors", "b": "other.safetensors"}}))
    assert sorted(SafetensorsReader(str(d)).names()) == ["a", "b"]
    # the index wins over a model.safetensors beside it
    write_safetensors(str(d / "model.safetensors"), {"c": torch.ones(1)})
    assert sorted(SafetensorsReader(str(d)).names()) == ["a", "b"]
    (d / "net.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"a": "weights.safetensors", "b": "gone.safetensors"}}))
    with pytest.raises(WeightError, match="gone.safetensors"):
        SafetensorsReader(str(d))
    (d / "net.safetensors.index.json").write_text(json.dumps({"weights": {}}))
    with pytest.raises(WeightError, match="unreadable shard index"):
        SafetensorsReader(str(d))


def test_broken_files_are_refused(tmp_path):
    with pytest.raises(WeightError, match="neither"):
        SafetensorsReader(str(tmp_path))
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(WeightError, match="too short"):
        SafetensorsReader(str(tmp_path))
    import struct
    hdr = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(WeightError, match="does not match"):
        SafetensorsReader(str(tmp_path))
    hdr = json.dumps({"a": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 4)
    with pytest.raises(WeightError, match="unsupported dtype"):
        SafetensorsReader(str(tmp_path))


def test_names_and_shapes_of_the_checkpoint():
    # crates/infer-worker/src/models/decoder.rs:237-385
    specs = build_llama(cfg_of("B")).param_specs()
    assert specs["model.embed_tokens.weight"].shape == (384, 160)
    assert specs["model.layers.2.self_attn.q_proj.weight"].shape == (160, 160)
    assert specs["model.layers.0.self_attn.k_proj.weight"].shape == (32, 160)
    assert specs["model.layers.0.self_attn.o_proj.weight"].shape == (160, 160)
    assert specs["model.layers.1.mlp.gate_proj.weight"].shape == (416, 160)
    assert specs["model.layers.1.mlp.down_proj.weight"].shape == (160, 416)
    assert specs["model.layers.1.post_attention_layernorm.weight"].shape == (160,)
    assert specs["model.norm.weight"].shape == (160,) and specs["lm_head.weight"].shape == (384, 160)
    assert len(specs) == 3 * 9 + 3
    assert "lm_head.weight" not in build_llama(cfg_of("A")).param_specs()        # tied


def test_one_error_lists_missing_unexpected_and_wrong(tmp_path):
    cfg = cfg_of("B")
    model = build_llama(cfg)
    tensors = dict(random_tensors(model, 0))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.ones(32)
    tensors["model.layers.2.self_attn.k_proj.weight"] = torch.ones(64, 160)
    tensors["model.layers.0.input_layernorm.weight"] = torch.ones(160, dtype=torch.int32)
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as e:
        check_checkpoint(model, SafetensorsReader(str(tmp_path)))
    msg = str(e.value)
    assert "missing tensors (2): model.layers.1.mlp.up_proj.weight, model.norm.weight" in msg
    assert "unexpected tensors (1): model.layers.0.self_attn.q_norm.weight" in msg
    assert "model.layers.2.self_attn.k_proj.weight: expected [32, 160], got [64, 160]" in msg
    assert "model.layers.0.input_layernorm.weight: expected floating point" in msg


def test_tied_head_contradictions(tmp_path):
    tied, untied = build_llama(cfg_of("A")), build_llama(cfg_of("B"))
    t = dict(random_tensors(tied, 0))
    t["lm_head.weight"] = torch.zeros(256, 64)
    write_safetensors(str(tmp_path / "model.safetensors"), t)
    with pytest.raises(WeightError, match="tie_word_embeddings=true but the checkpoint holds lm_head.weight"):
        check_checkpoint(tied, SafetensorsReader(str(tmp_path)))
    t = dict(random_tensors(untied, 0))
    del t["lm_head.weight"]
    write_safetensors(str(tmp_path / "model.safetensors"), t)
    with pytest.raises(WeightError, match="tie_word_embeddings=false but the checkpoint has no lm_head.weight"):
        check_checkpoint(untied, SafetensorsReader(str(tmp_path)))


def test_random_weights_mode(tmp_path):
    cfg = cfg_of("A")
    d1 = write_random_model(cfg, 0, str(tmp_path / "a"))
    d2 = write_random_model(cfg, 0, str(tmp_path / "b"))
    d3 = write_random_model(cfg, 1, str(tmp_path / "c"))
    assert sorted(os.listdir(d1)) == ["config.json", "model.safetensors"]
    assert LlamaConfig.from_dict(json.load(open(os.path.join(d1, "config.json")))) == cfg
    r1, r2, r3 = (SafetensorsReader(d) for d in (d1, d2, d3))
    check_checkpoint(build_llama(cfg), r1)
    for n in r1.names():
        assert torch.equal(r1.tensor(n), r2.tensor(n))                 # same seed, same bytes
        assert not torch.equal(r1.tensor(n), r3.tensor(n))             # another seed
        assert r1.tensor(n).dtype == torch.bfloat16
    w = r1.tensor("model.layers.0.mlp.down_proj.weight").float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    n = r1.tensor("model.norm.weight").float()
    assert abs(n.mean().item() - 1.0) < 0.02 and 0.005 < n.std().item() < 0.04
    # a tensor's values depend on its name and the seed only, not on what else the model holds
    big = dict(random_tensors(build_llama(cfg_of("A")), 0))
    assert torch.equal(big["model.embed_tokens.weight"], r1.tensor("model.embed_tokens.weight"))
    d4 = write_random_model(cfg, 0, str(tmp_path / "d"), dtype=torch.float32, norm_noise=False)
    r4 = SafetensorsReader(d4)
    assert r4.tensor("model.norm.weight").dtype == torch.float32
    assert torch.all(r4.tensor("model.norm.weight") == 1.0)


@pytest.mark.parametrize("stored", [torch.float16, torch.float32, torch.bfloat16])
def test_a_checkpoint_is_cast_once_from_its_stored_dtype(tmp_path, stored):
    """A float16 (or 32-bit) checkpoint in a float32 run keeps every stored bit: the parts hold
    exactly the stored values, not values rounded to bfloat16 on the way
    (crates/infer-worker/src/models/loader.rs:1398-1516).  In a bfloat16 run the values are the
    stored ones rounded once."""
    from rustinfer_amd.parts import Runtime
    from rustinfer_amd.weights import load_weights
    cfg = cfg_of("B")
    # values with more mantissa than bfloat16 holds
    src = {n: (t.float() * 1.2345).to(stored) for n, t in random_tensors(build_llama(cfg), 3, torch.float32)}
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg.to_dict(), f)
    write_safetensors(str(tmp_path / "model.safetensors"), src)
    assert SafetensorsReader(str(tmp_path)).tensor("model.norm.weight").dtype == stored
    for run in (torch.float32, torch.bfloat16):
        model = build_llama(cfg)
        load_weights(model, str(tmp_path), Runtime(torch.device("cpu"), run, None))
        att, mlp = model.layers[1].mixer, model.layers[1].ffn
        p = "model.layers.1."
        qkv = torch.cat([src[p + f"self_attn.{x}_proj.weight"] for x in "qkv"])
        pairs = [(att.qkv.weight, qkv), (att.o.weight, src[p + "self_attn.o_proj.weight"]),
                 (mlp.gate_up.weight, torch.cat([src[p + "mlp.gate_proj.weight"], src[p + "mlp.up_proj.weight"]])),
                 (mlp.down.weight, src[p + "mlp.down_proj.weight"]),
                 (model.embed.weight, src["model.embed_tokens.weight"]),
                 (model.lm_head.weight, src["lm_head.weight"])]
        for got, want in pairs:
            assert got.dtype == run and torch.equal(got, want.to(run))
            if run == torch.float32 and stored != torch.bfloat16:
                assert not torch.equal(got, want.to(torch.bfloat16).float())    # the test can tell the difference
        norm = model.layers[1].mixer_norm.weight
        want = src[p + "input_layernorm.weight"]
        assert norm.dtype == (torch.float32 if stored == torch.float32 else run)  # stored in 32-bit stays 32-bit
        assert torch.equal(norm, want.to(norm.dtype))


def test_a_spec_may_bring_its_own_distribution():
    """Random weights of a parameter that is neither a matrix nor a norm weight: the spec gives a
    normal distribution's mean and deviation or a function; a kind nobody knows is an error, not
    silently N(0, 0.02)."""
    from rustinfer_amd.parts import ParamSpec
    from rustinfer_amd.weights.random_init import random_tensor
    t = random_tensor("x.bias", ParamSpec((4000,), mean=3.0, std=0.5), 1, torch.float32)
    assert abs(t.mean().item() - 3.0) < 0.05 and abs(t.std().item() - 0.5) < 0.05
    t = random_tensor("x.scale", ParamSpec((4000,), mean=1.0), 1, torch.float32)          # deviation as for matrices
    assert abs(t.mean().item() - 1.0) < 0.01 and abs(t.std().item() - 0.02) < 0.005
    draw = lambda g, shape, device: 0.6 + 0.3 * torch.rand(shape, generator=g, device=device)
    a = random_tensor("x.decay", ParamSpec((64, 3), init=draw), 7, torch.bfloat16)
    b = random_tensor("x.decay", ParamSpec((64, 3), init=draw), 7, torch.bfloat16)
    assert a.dtype == torch.bfloat16 and torch.equal(a, b) and 0.6 <= a.min().item() and a.max().item() <= 0.9
    assert not torch.equal(a, random_tensor("y.decay", ParamSpec((64, 3), init=draw), 7, torch.bfloat16))
    with pytest.raises(ValueError, match="shape"):
        random_tensor("x", ParamSpec((3,), init=lambda g, shape, device: torch.zeros(4)), 0, torch.float32)
    with pytest.raises(ValueError, match="unknown kind"):
        random_tensor("x", ParamSpec((3,), kind="decay"), 0, torch.float32)


def test_tensors_made_when_asked_for_and_the_budget_of_second_copies():
    """``LazyTensors`` makes a tensor each time it is asked and narrows by prefix as a dictionary
    of names does; ``Runtime.tile`` stops making second copies when its budget is spent."""
    from types import SimpleNamespace
    from rustinfer_amd.parts.base import LazyTensors, Runtime, narrow_tensors
    made = []

    def make(name):
        made.append(name)
        return torch.full((2,), float(len(name)))

    names = {"layers.0.a.w": 1, "layers.0.b.w": 1, "layers.1.a.w": 1, "norm.w": 1}
    lazy = LazyTensors(names, make)
    assert made == [] and "norm.w" in lazy and "nope" not in lazy and len(lazy) == 4
    sub = narrow_tensors(narrow_tensors(lazy, "layers"), "0")
    assert sorted(sub.keys()) == ["a.w", "b.w"] and made == []
    assert torch.equal(sub["a.w"], torch.full((2,), 12.0)) and made == ["layers.0.a.w"]
    with pytest.raises(KeyError):
        sub["c.w"]
    plain = {n: torch.zeros(1) for n in names}
    assert sorted(narrow_tensors(narrow_tensors(plain, "layers"), "0")) == ["a.w", "b.w"]

    ops = SimpleNamespace(tile_weight=lambda w: w.clone() if w.shape[0] % 2 == 0 else None)
    rt = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=ops, tile_budget=100)
    w = torch.zeros(4, 4)                                    # 64 bytes
    assert rt.tile(w) is not None and rt.tile_budget == 36 and rt.tiled_bytes == 64
    assert rt.tile(w) is None and rt.tile_budget == 36      # does not fit any more
    assert rt.tile(torch.zeros(3, 2)) is None and rt.tile_budget == 36 and rt.tiled_bytes == 64   # no such form: given back
    assert rt.tile(torch.zeros(2, 4)) is not None and rt.tile_budget == 4
    free = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=ops)
    assert free.tile(w) is not None and free.tile_budget is None and free.tiled_bytes == 64
    off = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=ops, tiled_weight_copy=False)
    assert off.tile(w) is None and not off.take_tile_budget(1)
