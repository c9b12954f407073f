"""Weights by name: the writer and reader of the container, the random-weights
mode, and the one error that lists everything wrong with a folder
(/root/reference/crates/nnis-model/src/safetensors_loader.rs:1075-1157)."""

import json
import os
import shutil
import struct

import pytest
import torch

import nnis_amd
import nnis_amd.models  # noqa: F401
from configs import TINY_A, TINY_B, TINY_C
from nnis_amd.config import spec_from_config
from nnis_amd.errors import WeightError
from nnis_amd.models import DecoderModel
from nnis_amd.weights import SafetensorsFile, load_weights, write_safetensors


def _specs(config):
    return DecoderModel(spec_from_config(config)[1]).tensors()


def test_container_round_trip_against_the_package(tmp_path):
    from safetensors import safe_open

    tensors = [("a", torch.randn(3, 5)), ("b.c", torch.randn(7).to(torch.bfloat16)), ("i", torch.arange(6, dtype=torch.int32).view(2, 3))]
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, {"note": "t"})
    with safe_open(path, framework="pt") as handle:  # the package reads what we wrote
        for name, tensor in tensors:
            assert torch.equal(handle.get_tensor(name), tensor)
    ours = SafetensorsFile(path)
    assert ours.entries["b.c"] == ("BF16", (7,)) and ours.metadata == {"note": "t"}
    for name, tensor in tensors:
        assert torch.equal(ours.tensor(name), tensor)


def test_random_model_folder(model_dirs):
    for name, config in (("A", TINY_A), ("B", TINY_B), ("C", TINY_C)):
        folder = model_dirs[name]
        assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
        handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
        names = set(handle.names())
        assert ("lm_head.weight" in names) == (not config["tie_word_embeddings"])
        stored = "BF16" if config["torch_dtype"] == "bfloat16" else "F32"
        assert all(dtype == stored for dtype, _ in handle.entries.values())
        gain = handle.tensor("model.norm.weight").float()
        matrix = handle.tensor("model.layers.0.mlp.up_proj.weight").float()
        assert abs(gain.mean().item() - 1.0) < 0.01 and 0.005 < gain.std().item() < 0.02
        assert abs(matrix.mean().item()) < 0.002 and 0.017 < matrix.std().item() < 0.023


def test_random_weights_follow_the_seed(tmp_path):
    a, b, c = (str(tmp_path / n) for n in "abc")
    nnis_amd.write_random_model(a, TINY_A, 5)
    nnis_amd.write_random_model(b, TINY_A, 5)
    nnis_amd.write_random_model(c, TINY_A, 6)
    read = lambda d: open(os.path.join(d, "model.safetensors"), "rb").read()  # noqa: E731
    assert read(a) == read(b) and read(a) != read(c)


def test_load_keeps_stored_types_and_shares_a_tied_head(model_dirs):
    w = load_weights(model_dirs["A"], _specs(TINY_A), "cpu", widen_to_float32=False)
    assert all(t.dtype == torch.bfloat16 for t in w.values())
    assert w["lm_head.weight"].data_ptr() == w["model.embed_tokens.weight"].data_ptr()
    wide = load_weights(model_dirs["A"], _specs(TINY_A), "cpu", widen_to_float32=True)
    assert all(t.dtype == torch.float32 for t in wide.values())
    assert torch.equal(wide["model.norm.weight"], w["model.norm.weight"].float())  # widening is exact
    # stored in 32-bit stays so
    c = load_weights(model_dirs["C"], _specs(TINY_C), "cpu", widen_to_float32=False)
    assert all(t.dtype == torch.float32 for t in c.values())


def test_one_error_lists_everything(model_dirs, tmp_path):
    folder = str(tmp_path / "broken")
    shutil.copytree(model_dirs["B"], folder)
    handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = []
    for name in handle.names():
        tensor = handle.tensor(name).clone()
        if name == "model.layers.1.mlp.up_proj.weight":
            continue  # missing
        if name == "model.layers.0.self_attn.k_proj.weight":
            tensor = tensor[:, :-1].contiguous()  # wrong shape
        if name == "model.norm.weight":
            tensor = tensor.to(torch.float16)  # unsupported stored type
        tensors.append((name, tensor))
    tensors.append(("model.layers.7.extra.weight", torch.zeros(2)))  # unexpected
    tensors.append(("model.layers.0.self_attn.rotary_emb.inv_freq", torch.zeros(16)))  # a known buffer: ignored
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    spec = spec_from_config(TINY_B)[1]
    assert spec.ignored_tensor_suffixes == ("rotary_emb.inv_freq",)  # the Llama description names it, not the loader
    with pytest.raises(WeightError) as info:
        load_weights(folder, _specs(TINY_B), "cpu", widen_to_float32=False, ignored_suffixes=spec.ignored_tensor_suffixes)
    text = str(info.value)
    assert "missing tensors (1)" in text and "model.layers.1.mlp.up_proj.weight [256, 96]" in text
    assert "unexpected tensors (1)" in text and "model.layers.7.extra.weight" in text
    assert "wrong shapes (1)" in text and "expected [32, 96], file has [32, 95]" in text
    assert "wrong stored types (1)" in text and "F16" in text
    assert "inv_freq" not in text
    with pytest.raises(WeightError, match=r"unexpected tensors \(2\)"):  # a model that does not name the buffer does not know it
        load_weights(folder, _specs(TINY_B), "cpu", widen_to_float32=False)


def test_untied_model_without_head_is_an_error(model_dirs, tmp_path):
    folder = str(tmp_path / "nohead")
    shutil.copytree(model_dirs["B"], folder)
    handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(n, handle.tensor(n).clone()) for n in handle.names() if n != "lm_head.weight"])
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_weights(folder, _specs(TINY_B), "cpu", widen_to_float32=False)


def test_head_in_file_wins_when_tied(model_dirs, tmp_path):
    # /root/reference/crates/nnis-model/src/safetensors_loader.rs:755-786
    folder = str(tmp_path / "tiedhead")
    shutil.copytree(model_dirs["A"], folder)
    handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = [(n, handle.tensor(n).clone()) for n in handle.names()]
    head = torch.full((512, 64), 0.5, dtype=torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors + [("lm_head.weight", head)])
    w = load_weights(folder, _specs(TINY_A), "cpu", widen_to_float32=False)
    assert torch.equal(w["lm_head.weight"], head)


def test_folder_errors(model_dirs, tmp_path):
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(WeightError, match="neither"):
        load_weights(str(empty), _specs(TINY_A), "cpu", False)
    both = str(tmp_path / "both")
    shutil.copytree(model_dirs["A"], both)
    with open(os.path.join(both, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {}}, f)
    with pytest.raises(WeightError, match="both"):
        load_weights(both, _specs(TINY_A), "cpu", False)
    # shards named by an index; a path that leaves the folder is refused
    sharded = tmp_path / "sharded"
    sharded.mkdir()
    handle = SafetensorsFile(os.path.join(model_dirs["A"], "model.safetensors"))
    names = handle.names()
    half = len(names) // 2
    write_safetensors(str(sharded / "s1.safetensors"), [(n, handle.tensor(n).clone()) for n in names[:half]])
    write_safetensors(str(sharded / "s2.safetensors"), [(n, handle.tensor(n).clone()) for n in names[half:]])
    weight_map = {n: ("s1.safetensors" if i < half else "s2.safetensors") for i, n in enumerate(names)}
    (sharded / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    w = load_weights(str(sharded), _specs(TINY_A), "cpu", False)
    assert torch.equal(w["model.norm.weight"], handle.tensor("model.norm.weight"))
    (sharded / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": "../A/model.safetensors"}}))
    with pytest.raises(WeightError, match="leaves"):
        load_weights(str(sharded), _specs(TINY_A), "cpu", False)


def test_malformed_container(tmp_path):
    path = tmp_path / "bad.safetensors"
    path.write_bytes(b"\x01\x02")
    with pytest.raises(WeightError, match="too short"):
        SafetensorsFile(str(path))
    path.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(WeightError, match="header length"):
        SafetensorsFile(str(path))
    path.write_bytes(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(WeightError, match="malformed"):
        SafetensorsFile(str(path))
    header = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    path.write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 8)
    with pytest.raises(WeightError, match="does not fit"):
        SafetensorsFile(str(path))


def test_tables_of_integers_are_kept_as_int32(tmp_path):
    """A part may declare a table of integers (here a toy embedding that maps token ids through a table
    before the lookup): the random model holds it as I32, the loader keeps it int32 on the bfloat16 path
    and on the 32-bit path (which widens everything else), takes I64 too, and names a float in its place
    as a wrong type."""
    from dataclasses import dataclass

    from nnis_amd.config import register_architecture
    from nnis_amd.models import ModelSpec, ScheduleEntry
    from nnis_amd.parts import Part, TensorSpec, register_part

    class RemappedTable(Part):
        def __init__(self, vocab_size, width, weight, remap):
            self.vocab_size, self.width, self.weight_name, self.remap_name = vocab_size, width, weight, remap

        def tensors(self):
            return [TensorSpec(self.weight_name, (self.vocab_size, self.width)),
                    TensorSpec(self.remap_name, (self.vocab_size,), init="index", high=self.vocab_size)]

    @dataclass(frozen=True)
    class RemapConfig:
        raw: dict

        @classmethod
        def from_dict(cls, raw):
            return cls(dict(raw))

    def remap_spec(cfg):
        return ModelSpec(
            architecture="RemapToyForCausalLM", width=32, vocab_size=97, max_positions=64, stored_dtype="bfloat16",
            embedding={"kind": "remapped_table", "vocab_size": 97, "width": 32, "weight": "emb", "remap": "remap"},
            positions={},
            layers=[{"kind": "pre_norm", "width": 32,
                     "norm1": {"kind": "rms", "width": 32, "eps": 1e-5, "weight": "n1"},
                     "mixer": {"kind": "causal_attention", "width": 32, "heads": 2, "kv_heads": 1, "head_dim": 16, "position": None,
                               "q": "q", "k": "k", "v": "v", "o": "o"},
                     "norm2": {"kind": "rms", "width": 32, "eps": 1e-5, "weight": "n2"},
                     "feed_forward": {"kind": "gated", "width": 32, "inner": 48, "gate": "g", "up": "u", "down": "d"}}],
            schedule=[ScheduleEntry(0)],
            final_norm={"kind": "rms", "width": 32, "eps": 1e-5, "weight": "norm"},
            head={"kind": "linear", "vocab_size": 97, "width": 32, "weight": "head", "tied_to": "emb"},
            config_json=cfg.raw)

    register_part("embedding", "remapped_table", RemappedTable, replace=True)
    register_architecture("RemapToyForCausalLM", RemapConfig, remap_spec, replace=True)
    folder = str(tmp_path / "remap")
    raw = {"architectures": ["RemapToyForCausalLM"], "model_type": "remap_toy"}
    nnis_amd.write_random_model(folder, raw, seed=4)
    stored = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    assert stored.entries["remap"] == ("I32", (97,)) and stored.entries["emb"][0] == "BF16"
    table = stored.tensor("remap").clone()
    everything = {name: stored.tensor(name).clone() for name in stored.names()}
    stored.close()
    assert table.dtype == torch.int32 and 0 <= int(table.min()) and int(table.max()) < 97 and len(set(table.tolist())) > 20
    specs = DecoderModel(spec_from_config(raw)[1]).tensors()
    for widen in (False, True):
        loaded = load_weights(folder, specs, "cpu", widen_to_float32=widen)
        assert loaded["remap"].dtype == torch.int32 and torch.equal(loaded["remap"], table)
        assert loaded["emb"].dtype == (torch.float32 if widen else torch.bfloat16)
    # stored in 64 bits: taken, narrowed; a value that does not fit is refused
    wide = dict(everything, remap=table.to(torch.int64))
    write_safetensors(os.path.join(folder, "model.safetensors"), wide.items())
    assert torch.equal(load_weights(folder, specs, "cpu", widen_to_float32=False)["remap"], table)
    wide["remap"][3] = 1 << 40
    write_safetensors(os.path.join(folder, "model.safetensors"), wide.items())
    with pytest.raises(WeightError, match="does not fit"):
        load_weights(folder, specs, "cpu", widen_to_float32=False)
    # a float where the table of integers should be, and integers where a matrix should be
    write_safetensors(os.path.join(folder, "model.safetensors"), dict(everything, remap=table.float()).items())
    with pytest.raises(WeightError, match="remap: stored as F32; a table of integers"):
        load_weights(folder, specs, "cpu", widen_to_float32=False)
    write_safetensors(os.path.join(folder, "model.safetensors"), dict(everything, norm=torch.ones(32, dtype=torch.int32)).items())
    with pytest.raises(WeightError, match="norm: stored as I32; supported are F32 and BF16"):
        load_weights(folder, specs, "cpu", widen_to_float32=False)


def test_stored_types_must_be_the_declared_one(model_dirs, tmp_path, capsys):
    """Every tensor is stored in config.json's torch_dtype
    (/root/reference/crates/nnis-model/src/safetensors_loader.rs:718-724); nothing is narrowed unless the
    caller says so (safetensors_loader.rs:610-624), and then to the nearest bfloat16, ties to even."""
    folder = str(tmp_path / "mixed")
    shutil.copytree(model_dirs["A"], folder)
    handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = [(n, handle.tensor(n).clone().float() if n == "model.norm.weight" else handle.tensor(n).clone()) for n in handle.names()]
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.raises(WeightError) as info:
        load_weights(folder, _specs(TINY_A), "cpu", widen_to_float32=False, declared_dtype="bfloat16")
    assert "wrong stored types (1)" in str(info.value) and "model.norm.weight: stored as F32; config.json declares bfloat16" in str(info.value)
    load_weights(folder, _specs(TINY_A), "cpu", widen_to_float32=False)  # without a declaration the mix is taken as stored
    with pytest.raises(WeightError, match="declares torch_dtype"):
        load_weights(folder, _specs(TINY_A), "cpu", False, declared_dtype="float16")

    # a 32-bit checkpoint: stays 32-bit (and says so), widens to itself, narrows only when asked
    capsys.readouterr()
    kept = load_weights(model_dirs["C"], _specs(TINY_C), "cpu", widen_to_float32=False, declared_dtype="float32")
    assert all(t.dtype == torch.float32 for t in kept.values())
    assert "stay so" in capsys.readouterr().err
    narrowed = load_weights(model_dirs["C"], _specs(TINY_C), "cpu", widen_to_float32=False, declared_dtype="float32",
                            narrow_to_bfloat16=True)
    assert capsys.readouterr().err == ""
    assert all(t.dtype == torch.bfloat16 for t in narrowed.values())
    name = "model.layers.0.mlp.up_proj.weight"
    # nearest, ties to even, worked on the bits: add 0x7fff + the kept part's lowest bit, drop the low half
    bits = kept[name].view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    want = (((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF).to(torch.int32)
    assert torch.equal(narrowed[name].view(torch.int16).to(torch.int32) & 0xFFFF, want)
    with pytest.raises(WeightError, match="bfloat16 runtime"):
        load_weights(model_dirs["C"], _specs(TINY_C), "cpu", widen_to_float32=True, narrow_to_bfloat16=True)


def test_init_rules_are_a_registry(tmp_path):
    from nnis_amd.errors import InvalidInput
    from nnis_amd.parts.base import TensorSpec
    from nnis_amd.weights.random_init import _INIT_RULES, register_init_rule, registered_init_rules

    assert {"matrix", "gain", "zeros", "index"} <= set(registered_init_rules())
    with pytest.raises(InvalidInput, match="already registered"):
        register_init_rule("matrix", lambda spec, generator, dtype: None)
    register_init_rule("test_sevens", lambda spec, generator, dtype: torch.full(tuple(spec.shape), 7.0, dtype=dtype))
    try:
        generator = torch.Generator().manual_seed(0)
        drawn = _INIT_RULES["test_sevens"](TensorSpec("x", (2, 3), init="test_sevens"), generator, torch.bfloat16)
        assert drawn.dtype == torch.bfloat16 and bool((drawn == 7).all())
        zeros = _INIT_RULES["zeros"](TensorSpec("b", (4,), init="zeros"), generator, torch.float32)
        assert zeros.dtype == torch.float32 and not zeros.any()
    finally:
        del _INIT_RULES["test_sevens"]
