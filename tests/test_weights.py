"""Weights: reading by name, element types, the one error that lists everything, random-weights mode."""
import json
import os
import struct

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY_A, TINY_B, make_model_folder

from lmsf_amd.config import LlamaConfig, get_architecture
from lmsf_amd.models import DecoderModel
from lmsf_amd.parts import Runtime
from lmsf_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError, declared_tensors, list_weight_files,
                              load_weights, write_random_model, write_safetensors)


def cpu_model(cfg, dtype=torch.float32):
    rt = Runtime(ops=None, device=torch.device("cpu"), dtype=dtype, max_positions=cfg.max_position_embeddings)
    return DecoderModel(get_architecture(cfg.architecture).build_spec(cfg), rt)


def rewrite(folder, change):
    """Load model.safetensors, let ``change`` edit the dict of tensors, write it back."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    change(tensors)
    save_file(tensors, path)


def test_declared_names_and_shapes_follow_the_configuration():
    cfg = LlamaConfig.from_dict(TINY_B)
    decls = declared_tensors(get_architecture(cfg.architecture), cfg)
    assert decls["model.embed_tokens.weight"].shape == (1000, 128)
    assert decls["model.layers.2.self_attn.q_proj.weight"].shape == (8 * 32, 128)
    assert decls["model.layers.0.self_attn.k_proj.weight"].shape == (1 * 32, 128)
    assert decls["model.layers.0.self_attn.k_proj.bias"].shape == (32,)
    assert decls["model.layers.1.self_attn.o_proj.weight"].shape == (128, 256)
    assert decls["model.layers.1.self_attn.o_proj.bias"].shape == (128,)
    assert decls["model.layers.1.mlp.gate_proj.weight"].shape == (352, 128)
    assert decls["model.layers.1.mlp.down_proj.weight"].shape == (128, 352)
    assert decls["model.layers.1.input_layernorm.weight"].shape == (128,) and decls["model.norm.weight"].init == "ones"
    assert decls["lm_head.weight"].shape == (1000, 128)
    assert "model.layers.3.mlp.up_proj.weight" not in decls and "model.layers.0.mlp.up_proj.bias" not in decls
    tied = declared_tensors(get_architecture("LlamaForCausalLM"), LlamaConfig.from_dict(TINY_A))
    assert "lm_head.weight" not in tied and "model.layers.0.self_attn.q_proj.bias" not in tied


def test_written_folder_is_read_by_the_safetensors_package_and_back(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "B")
    theirs = load_file(os.path.join(folder, "model.safetensors"))
    ours = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    assert set(theirs) == set(ours.entries)
    for name in ("model.embed_tokens.weight", "model.layers.1.self_attn.v_proj.bias"):
        assert torch.equal(theirs[name], ours.read(name))
    ours.close()
    with open(os.path.join(folder, "config.json")) as f:
        assert LlamaConfig.from_dict(json.load(f)) == cfg
    # same seed, same values; another seed, other values; norm weights are ones
    again, _ = make_model_folder(tmp_path / "again", "B")
    other, _ = make_model_folder(tmp_path / "other", "B", seed=5)
    t2, t3 = load_file(os.path.join(again, "model.safetensors")), load_file(os.path.join(other, "model.safetensors"))
    assert all(torch.equal(theirs[k], t2[k]) for k in theirs)
    assert not torch.equal(theirs["lm_head.weight"], t3["lm_head.weight"])
    assert torch.equal(theirs["model.norm.weight"], torch.ones(128))
    w = theirs["model.layers.0.mlp.up_proj.weight"]
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002


def test_reader_takes_every_storage_type_and_refuses_a_header_that_lies(tmp_path):
    """The reader is C++ (csrc/host/safetensors.cc): a file of every dtype written by the safetensors package is
    read back to the bit, also tensors of no elements and of no dimensions; headers whose entries overlap, repeat a
    name, claim more bytes than their shape holds or more than the file has are refused, each by name."""
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(3)
    tensors = {
        "f32": torch.randn(3, 5, generator=g), "bf16": torch.randn(7, generator=g).bfloat16(),
        "f16": torch.randn(2, 3, 4, generator=g).half(), "f64": torch.randn(2, generator=g).double(),
        "i64": torch.arange(5), "i32": torch.arange(6, dtype=torch.int32).reshape(2, 3),
        "i16": torch.arange(4, dtype=torch.int16), "i8": torch.arange(3, dtype=torch.int8),
        "u8": torch.arange(9, dtype=torch.uint8), "flag": torch.tensor([True, False, True]),
        "none": torch.zeros(0, 4), "scalar": torch.tensor(2.5),
    }
    path = str(tmp_path / "all.safetensors")
    save_file(tensors, path)
    f = SafetensorsFile(path)
    assert set(f.entries) == set(tensors)
    for name, t in tensors.items():
        got = f.read(name)
        assert got.dtype == t.dtype and got.shape == t.shape and torch.equal(got, t), name
    kept = f.read("f32")
    over_the_file = f.read("bf16", copy=False)       # (a tensor over the mapping: gone before the file closes)
    assert torch.equal(over_the_file, tensors["bf16"])
    del over_the_file
    f.close()
    assert torch.equal(kept, tensors["f32"])          # (a tensor read owns its memory)

    def file_with(header: dict, data: bytes = bytes(64)) -> str:
        text = json.dumps(header).encode()
        bad = str(tmp_path / "bad.safetensors")
        with open(bad, "wb") as out:
            out.write(struct.pack("<Q", len(text)) + text + data)
        return bad
    entry = lambda dtype, shape, a, b: {"dtype": dtype, "shape": shape, "data_offsets": [a, b]}   # noqa: E731
    for header, what in (
            ({"a": entry("U8", [8], 0, 8), "b": entry("U8", [8], 4, 12)}, "overlap"),
            ({"a": entry("F32", [2, 2], 0, 12)}, "12 bytes for shape"),
            ({"a": entry("F32", [2, 2], 56, 72)}, "outside the file"),
            ({"a": entry("F8_E4M3", [4], 0, 4)}, "unsupported dtype"),
            ({"a": entry("U8", [-4], 0, 4)}, "malformed header entry"),
            ({"a": {"dtype": "U8", "shape": [4]}}, "malformed header entry"),
            ({"a": [1, 2]}, "malformed header entry"),
            ({"a": entry("U8", [1] * 9, 0, 1)}, "9 dimensions")):
        with pytest.raises(SafetensorsError, match=what):
            SafetensorsFile(file_with(header))
    twice = b'{"a": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}, "a": {"dtype": "U8", "shape": [4], "data_offsets": [4, 8]}}'
    with open(str(tmp_path / "twice.safetensors"), "wb") as out:
        out.write(struct.pack("<Q", len(twice)) + twice + bytes(8))
    with pytest.raises(SafetensorsError, match="listed twice"):
        SafetensorsFile(str(tmp_path / "twice.safetensors"))
    with open(str(tmp_path / "text.safetensors"), "wb") as out:
        out.write(struct.pack("<Q", 5) + b"{nope")
    with pytest.raises(SafetensorsError, match="not valid JSON"):
        SafetensorsFile(str(tmp_path / "text.safetensors"))
    with pytest.raises(SafetensorsError, match="cannot be opened"):
        SafetensorsFile(str(tmp_path / "absent.safetensors"))


def test_fused_rows_and_tied_head(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "B")
    model = cpu_model(cfg)
    load_weights(model.parts(), folder, torch.device("cpu"), torch.float32)
    raw = load_file(os.path.join(folder, "model.safetensors"))
    att = model.blocks[1].mixer
    p = "model.layers.1.self_attn."
    assert torch.equal(att.qkv.weight, torch.cat([raw[p + "q_proj.weight"], raw[p + "k_proj.weight"],
                                                  raw[p + "v_proj.weight"]]))
    assert torch.equal(att.qkv.bias, torch.cat([raw[p + "q_proj.bias"], raw[p + "k_proj.bias"], raw[p + "v_proj.bias"]]))
    ffn = model.blocks[1].feed_forward
    assert torch.equal(ffn.gate_up.weight, torch.cat([raw["model.layers.1.mlp.gate_proj.weight"],
                                                      raw["model.layers.1.mlp.up_proj.weight"]]))
    folder_a, cfg_a = make_model_folder(tmp_path, "A")
    tied = cpu_model(cfg_a)
    load_weights(tied.parts(), folder_a, torch.device("cpu"), torch.float32)
    assert tied.head.weight.data_ptr() == tied.embedding.weight.data_ptr()


def test_element_types(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "A", dtype="bfloat16")
    rewrite(folder, lambda t: t.update({"model.norm.weight": t["model.norm.weight"].float(),
                                        "model.layers.0.mlp.down_proj.weight":
                                            t["model.layers.0.mlp.down_proj.weight"].half()}))
    m16 = cpu_model(cfg, torch.bfloat16)
    load_weights(m16.parts(), folder, torch.device("cpu"), torch.bfloat16)
    assert m16.embedding.weight.dtype == torch.bfloat16
    assert m16.final_norm.weight.dtype == torch.float32                       # stored in 32 bits: stays so
    assert m16.blocks[0].feed_forward.down.weight.dtype == torch.bfloat16     # float16 storage is converted
    m32 = cpu_model(cfg, torch.float32)
    load_weights(m32.parts(), folder, torch.device("cpu"), torch.float32)
    assert all(p.weight.dtype == torch.float32 for p in m32.parts() if getattr(p, "weight", None) is not None)
    rewrite(folder, lambda t: t.update({"model.norm.weight": torch.ones(64, dtype=torch.int32)}))
    with pytest.raises(WeightsError, match="model.norm.weight.*stored as torch.int32"):
        load_weights(cpu_model(cfg).parts(), folder, torch.device("cpu"), torch.float32)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "B")

    def damage(t):
        del t["model.layers.0.self_attn.q_proj.weight"]
        del t["model.layers.2.mlp.down_proj.weight"]
        t["model.layers.1.mlp.up_proj.weight"] = torch.zeros(352, 127)
        t["model.norm.weight"] = torch.zeros(2, 64)
        t["model.layers.7.input_layernorm.weight"] = torch.zeros(128)
        t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)   # tolerated: old exports carry it

    rewrite(folder, damage)
    with pytest.raises(WeightsError) as e:
        load_weights(cpu_model(cfg).parts(), folder, torch.device("cpu"), torch.float32,
                     tolerated=get_architecture(cfg.architecture).tolerated_tensors)
    err = e.value
    assert err.missing == ["model.layers.0.self_attn.q_proj.weight", "model.layers.2.mlp.down_proj.weight"]
    assert err.unexpected == ["model.layers.7.input_layernorm.weight"]
    assert err.wrong_shape == [("model.layers.1.mlp.up_proj.weight", (352, 128), (352, 127)),
                               ("model.norm.weight", (128,), (2, 64))]
    text = str(err)
    for word in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "q_proj.weight",
                 "expected [352, 128] found [352, 127]", folder):
        assert word in text
    assert "rotary_emb" not in text


def test_tied_checkpoint_may_carry_a_head(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "A")
    rewrite(folder, lambda t: t.update({"lm_head.weight": t["model.embed_tokens.weight"].clone()}))
    load_weights(cpu_model(cfg).parts(), folder, torch.device("cpu"), torch.float32,
                 tolerated=get_architecture(cfg.architecture).tolerated_tensors)
    with pytest.raises(WeightsError, match="unexpected tensors"):
        load_weights(cpu_model(cfg).parts(), folder, torch.device("cpu"), torch.float32)


def test_shards_with_index_equal_one_file(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "A")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    names = sorted(tensors)
    shard = str(tmp_path / "sharded")
    os.makedirs(shard)
    halves = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    for fname, ns in halves.items():
        write_safetensors(os.path.join(shard, fname), [(n, tensors[n]) for n in ns])
    with open(os.path.join(shard, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {n: fname for fname, ns in halves.items() for n in ns}}, f)
    assert [os.path.basename(p) for p in list_weight_files(shard)] == sorted(halves)
    a, b = cpu_model(cfg), cpu_model(cfg)
    load_weights(a.parts(), folder, torch.device("cpu"), torch.float32)
    load_weights(b.parts(), shard, torch.device("cpu"), torch.float32)
    assert torch.equal(a.blocks[1].mixer.qkv.weight, b.blocks[1].mixer.qkv.weight)
    os.unlink(os.path.join(shard, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightsError, match="not there"):
        load_weights(cpu_model(cfg).parts(), shard, torch.device("cpu"), torch.float32)


def test_broken_files_are_refused(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "A")
    path = os.path.join(folder, "model.safetensors")
    data = open(path, "rb").read()
    with open(path, "wb") as f:
        f.write(data[:len(data) - 100])
    with pytest.raises(WeightsError, match="truncated"):
        load_weights(cpu_model(cfg).parts(), folder, torch.device("cpu"), torch.float32)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(path)
    os.unlink(path)
    with pytest.raises(WeightsError, match="no safetensors file"):
        load_weights(cpu_model(cfg).parts(), folder, torch.device("cpu"), torch.float32)


def test_write_random_model_uses_the_requested_storage(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_A)
    folder = write_random_model(str(tmp_path / "bf"), cfg, seed=3, dtype="bfloat16")
    t = load_file(os.path.join(folder, "model.safetensors"))
    assert all(v.dtype == torch.bfloat16 for v in t.values())
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f)["torch_dtype"] == "bfloat16"


def test_loading_keeps_one_source_tensor_alive_beside_the_weights(tmp_path):
    """The fused products copy every checkpoint tensor into its rows of one buffer and drop it at once, and
    the loader keeps nothing but tied tensors: while the model loads, at most one tensor that is not part of
    the model is alive."""
    import gc
    import weakref
    from lmsf_amd.weights.loader import load_weights_from_generator
    folder, cfg = make_model_folder(tmp_path, "B")
    raw = load_file(os.path.join(folder, "model.safetensors"))
    model = cpu_model(cfg)
    made = []                 # (name, weak reference) of everything handed out
    most = [0]

    def make(name, decl):
        gc.collect()
        alive = [n for n, r in made if r() is not None and not _is_model_tensor(model, r())]
        most[0] = max(most[0], len(alive))
        t = raw[name].clone()
        made.append((name, weakref.ref(t)))
        return t

    load_weights_from_generator(model.parts(), make)
    assert most[0] <= 1, most[0]
    p = "model.layers.2.self_attn."
    assert torch.equal(model.blocks[2].mixer.qkv.weight,
                       torch.cat([raw[p + "q_proj.weight"], raw[p + "k_proj.weight"], raw[p + "v_proj.weight"]]))
    # mixed storage: the buffer takes the widest element type
    wide = cpu_model(cfg, torch.bfloat16)
    load_weights_from_generator(wide.parts(), lambda n, d: raw[n].clone() if n.endswith("k_proj.weight")
                                else raw[n].to(torch.bfloat16))
    assert wide.blocks[0].mixer.qkv.weight.dtype == torch.float32
    assert torch.equal(wide.blocks[0].mixer.qkv.weight[256:288], raw["model.layers.0.self_attn.k_proj.weight"])


def test_weight_rows_lie_as_far_apart_as_the_kernels_ask(tmp_path):
    """The kernel object says how many elements to leave between two rows of a linear layer's weight; fused and
    single matrices, and buffers that widen to 32 bits on the way, are laid out so, and hold the checkpoint's
    values."""
    from types import SimpleNamespace
    from lmsf_amd.weights.loader import load_weights_from_generator
    folder, cfg = make_model_folder(tmp_path, "B")
    raw = load_file(os.path.join(folder, "model.safetensors"))
    ops = SimpleNamespace(weight_row_pad=lambda in_features, dtype: 24 if dtype == torch.bfloat16 else 12)
    rt = Runtime(ops=ops, device=torch.device("cpu"), dtype=torch.bfloat16, max_positions=cfg.max_position_embeddings)
    model = DecoderModel(get_architecture(cfg.architecture).build_spec(cfg), rt)
    load_weights_from_generator(model.parts(), lambda n, d: raw[n].clone() if n.endswith("layers.1.self_attn.v_proj.weight")
                                else raw[n].to(torch.bfloat16))
    p = "model.layers.0."
    qkv, down = model.blocks[0].mixer.qkv.weight, model.blocks[0].feed_forward.down.weight
    assert qkv.stride() == (qkv.shape[1] + 24, 1) and down.stride() == (down.shape[1] + 24, 1)
    assert torch.equal(qkv, torch.cat([raw[p + "self_attn.%s_proj.weight" % n] for n in "qkv"]).to(torch.bfloat16))
    assert torch.equal(down, raw[p + "mlp.down_proj.weight"].to(torch.bfloat16))
    assert model.blocks[0].mixer.qkv.bias.is_contiguous()
    wide = model.blocks[1].mixer.qkv.weight       # its last source is stored in 32 bits
    assert wide.dtype == torch.float32 and wide.stride() == (wide.shape[1] + 12, 1)
    p = "model.layers.1.self_attn."
    assert torch.equal(wide, torch.cat([raw[p + "q_proj.weight"].to(torch.bfloat16).float(),
                                        raw[p + "k_proj.weight"].to(torch.bfloat16).float(), raw[p + "v_proj.weight"]]))


def _is_model_tensor(model, t):
    return any(getattr(p, a, None) is not None and getattr(p, a).data_ptr() == t.data_ptr()
               for p in model.parts() for a in ("weight", "bias"))


def test_matrices_stored_in_32_bits_are_cast_to_the_run_type_at_load(tmp_path):
    """A float32 checkpoint in a bfloat16 run: the matrices are cast as the reference casts at load
    (core/src/model_executor/models/model_factory.rs:124-139), the norms' weights keep their 32 bits; on request
    the matrices stay as stored, and that is reported."""
    import warnings
    folder, cfg = make_model_folder(tmp_path, "A", dtype="float32")
    m = cpu_model(cfg, torch.bfloat16)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        load_weights(m.parts(), folder, torch.device("cpu"), torch.bfloat16)
    for part in m.parts():
        w = getattr(part, "weight", None)
        if w is not None:
            assert w.dtype == (torch.float32 if w.dim() == 1 else torch.bfloat16), part.prefix
    raw = load_file(os.path.join(folder, "model.safetensors"))
    assert torch.equal(m.blocks[0].feed_forward.down.weight, raw["model.layers.0.mlp.down_proj.weight"].to(torch.bfloat16))
    kept = cpu_model(cfg, torch.bfloat16)
    with pytest.warns(UserWarning, match="stored in 32 bits"):
        load_weights(kept.parts(), folder, torch.device("cpu"), torch.bfloat16, keep_float32=True)
    assert kept.blocks[0].mixer.qkv.weight.dtype == torch.float32
