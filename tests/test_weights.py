"""Weights: the safetensors reader's rules, the by-name check with its one error, the random-weights mode."""

import json
import struct

import pytest
import torch

from helpers import TINY_A, INIT_A, model_folder
from llmx_amd import MiniMaxM3Config, RandomInit, WeightsError
from llmx_amd.parts.spec import TensorSpec
from llmx_amd.weights import ModelFiles, SafetensorsError, SafetensorsFile, check, device_dtype, host_values, load, write_safetensors
from llmx_amd.weights.folder import model_tensor_specs, random_tensors, write_random_model


def test_written_file_reads_back(tmp_path):
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).view(2, 3),
               "empty": torch.zeros(0, 4)}
    write_safetensors(tmp_path / "x.safetensors", tensors, {"note": "t"})
    f = SafetensorsFile(tmp_path / "x.safetensors")
    assert set(f.names()) == set(tensors) and f.metadata == {"note": "t"}
    for n, t in tensors.items():
        got = f.tensor(n)
        assert got.dtype == t.dtype and tuple(got.shape) == tuple(t.shape) and torch.equal(got, t)
    # the safetensors package reads the same file
    from safetensors import safe_open
    with safe_open(str(tmp_path / "x.safetensors"), framework="pt") as g:
        assert torch.equal(g.get_tensor("b"), tensors["b"])


def raw_file(path, header, data: bytes, pad_to: int = 8):
    """A file with this header (a dict, or JSON text as it stands) padded with spaces so that the data area begins at
    a multiple of `pad_to` bytes."""
    blob = header.encode() if isinstance(header, str) else json.dumps(header).encode()
    while (8 + len(blob)) % pad_to:
        blob += b" "
    path.write_bytes(struct.pack("<Q", len(blob)) + blob + data)


@pytest.mark.parametrize("header,data,text", [
    ({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8], "extra": 1}}, b"\0" * 8, "exactly dtype, shape and data_offsets"),
    ({"t": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}, b"\0" * 2, "has dtype F8_E4M3, which this engine does not read"),
    ({"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8, "do not span its shape"),
    ({"t": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12, "gap or an overlap"),
    ({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 12, "does not end where its last tensor ends"),
    ({"t": {"dtype": "F32", "shape": [2, -1], "data_offsets": [0, 8]}}, b"\0" * 8, "invalid shape"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}, "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12,
     "gap or an overlap"),
])
def test_reader_refusals(tmp_path, header, data, text):
    raw_file(tmp_path / "bad.safetensors", header, data)
    with pytest.raises(SafetensorsError, match=text):
        SafetensorsFile(tmp_path / "bad.safetensors")


def test_a_key_twice_in_the_header_is_refused(tmp_path):
    """The standard JSON parser would silently keep the last of two equal keys
    (/root/reference/src/format/safetensors.hpp:40-44,69,109 refuse them)."""
    entry = '{"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}'
    raw_file(tmp_path / "twice.safetensors", '{"t": %s, "t": %s}' % (entry, entry), b"\0" * 8)
    with pytest.raises(SafetensorsError, match="header of .*twice.safetensors repeats key t"):
        SafetensorsFile(tmp_path / "twice.safetensors")
    raw_file(tmp_path / "inner.safetensors", '{"t": {"dtype": "F32", "dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}', b"\0" * 8)
    with pytest.raises(SafetensorsError, match="repeats key dtype"):
        SafetensorsFile(tmp_path / "inner.safetensors")


def test_metadata_must_be_an_object_of_strings(tmp_path):
    entry = {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}
    raw_file(tmp_path / "m1.safetensors", {"__metadata__": {"format": "pt", "step": 3}, "t": entry}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="__metadata__ value of step .* is not a string"):
        SafetensorsFile(tmp_path / "m1.safetensors")
    raw_file(tmp_path / "m2.safetensors", {"__metadata__": ["pt"], "t": entry}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="__metadata__ of .* is not an object"):
        SafetensorsFile(tmp_path / "m2.safetensors")


def test_a_tensor_at_an_unaligned_file_offset_is_refused(tmp_path):
    """Elements must lie at multiples of their size (of 4 bytes at most) in the file, so that the map can be read in place
    (/root/reference/src/format/safetensors.hpp:123-126)."""
    # a bfloat16 tensor of 3 elements pushes the float32 tensor behind it to an offset of 6
    header = {"h": {"dtype": "BF16", "shape": [3], "data_offsets": [0, 6]}, "f": {"dtype": "F32", "shape": [2], "data_offsets": [6, 14]}}
    raw_file(tmp_path / "odd.safetensors", header, b"\0" * 14)
    with pytest.raises(SafetensorsError, match="tensor f is not at a 4-byte-aligned file offset"):
        SafetensorsFile(tmp_path / "odd.safetensors")
    # the same tensors with the data area one byte off: the bfloat16 tensor is the first to be refused
    raw_file(tmp_path / "off.safetensors", {"h": {"dtype": "BF16", "shape": [3], "data_offsets": [0, 6]}}, b"\0" * 6, pad_to=1)
    if (8 + len(json.dumps({"h": {"dtype": "BF16", "shape": [3], "data_offsets": [0, 6]}}))) % 2:
        with pytest.raises(SafetensorsError, match="tensor h is not at a 2-byte-aligned file offset"):
            SafetensorsFile(tmp_path / "off.safetensors")
    # the writer orders wider elements first, so what it writes is always aligned
    write_safetensors(tmp_path / "ok.safetensors", {"h": torch.zeros(3, dtype=torch.bfloat16), "f": torch.ones(2), "i": torch.zeros(1, dtype=torch.int64)})
    f = SafetensorsFile(tmp_path / "ok.safetensors")
    assert f.entries["i"].begin == 0 and f.entries["f"].begin == 8 and f.entries["h"].begin == 16 and torch.equal(f.tensor("f"), torch.ones(2))


def test_an_index_that_names_a_file_outside_its_folder_is_refused(tmp_path):
    """/root/reference/src/format/safetensors.hpp:134-137: a file named by an index sits beside it."""
    write_safetensors(tmp_path / "part.safetensors", {"t": torch.zeros(2)})
    for bad in ("../part.safetensors", "sub/part.safetensors", "..", ""):
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"t": bad}}))
        with pytest.raises(WeightsError, match="names a file outside its directory"):
            ModelFiles(tmp_path)
    (tmp_path / "model.safetensors.index.json").write_text('{"weight_map": {"t": "part.safetensors", "t": "part.safetensors"}}')
    with pytest.raises(SafetensorsError, match="repeats key t"):
        ModelFiles(tmp_path)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"t": 3}}))
    with pytest.raises(WeightsError, match="weight_map value of t is not a file name"):
        ModelFiles(tmp_path)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"t": "part.safetensors"}}))
    assert list(ModelFiles(tmp_path).names()) == ["t"]


def test_header_longer_than_file(tmp_path):
    (tmp_path / "bad.safetensors").write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="beyond the file or the limit"):
        SafetensorsFile(tmp_path / "bad.safetensors")


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = MiniMaxM3Config(**TINY_A)
    tensors = random_tensors(cfg, INIT_A)
    del tensors["model.layers.1.self_attn.o_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.shared_experts.down_proj.weight"] = torch.zeros(4, 4)
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16)          # the per-head width, not the projection's
    tensors["model.layers.0.mlp.gate.e_score_correction_bias"] = torch.zeros(8, dtype=torch.int32)
    folder = tmp_path / "m"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg.to_json()))
    write_safetensors(folder / "model.safetensors", tensors)
    files = ModelFiles(folder)
    with pytest.raises(WeightsError) as err:
        load(model_tensor_specs(cfg), files, torch.device("cpu"), exact=True)
    e = err.value
    assert e.missing == ["model.layers.1.self_attn.o_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.mlp.shared_experts.down_proj.weight"]
    assert e.wrong_shape == [("model.layers.0.self_attn.q_norm.weight", (16,), (64,))]
    assert e.wrong_type == [("model.layers.0.mlp.gate.e_score_correction_bias", "torch.int32")]
    text = str(e)
    for name in e.missing + e.unexpected:
        assert name in text
    assert "is [16], expected [64]" in text


def test_types_on_the_device():
    m, n, r, i = (TensorSpec("x", (2, 2), role) for role in ("matrix", "norm", "router", "int"))
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert device_dtype(m, bf, exact=False) == bf          # bfloat16 stays bfloat16
    assert device_dtype(m, f32, exact=False) == f32        # a tensor stored in 32 bits stays so
    assert device_dtype(m, f16, exact=False) == f32        # half is widened, exactly
    assert device_dtype(m, bf, exact=True) == f32          # the 32-bit path widens everything
    assert device_dtype(n, bf, exact=False) == f32 and device_dtype(r, bf, exact=False) == f32
    assert device_dtype(i, torch.int64, exact=False) == torch.int32
    # a type the spec states holds in both paths, whatever the file stores
    decay = TensorSpec("d", (4,), "matrix", dtype="float32")
    assert device_dtype(decay, bf, exact=False) == f32 and device_dtype(TensorSpec("t", (4,), "table", dtype="bfloat16"), f32, exact=True) == bf
    with pytest.raises(ValueError, match="dtype 'float16' is not one of"):
        TensorSpec("x", (1,), dtype="float16")
    with pytest.raises(ValueError, match="role 'gate' is not one of"):
        TensorSpec("x", (1,), "gate")
    with pytest.raises(ValueError, match="init .* is not"):
        TensorSpec("x", (1,), init=("lognormal", 0, 1))


def test_a_spec_states_how_random_weights_fill_it():
    """A parameter of a kind the roles do not know brings its own distribution; the run's RandomInit does not touch it."""
    from llmx_amd.weights.random_init import distribution, stored_dtype
    init = RandomInit(seed=3, std=0.02, norm_std=0.1, bias_range=0.5)
    u = TensorSpec("layer.decay", (4096,), "matrix", dtype="float32", init=("uniform", 0.9, 0.999))
    assert distribution(u, init) == (1, 0.9, 0.999) and stored_dtype(u, init) == torch.float32
    v = host_values(u, init)
    assert v.dtype == torch.float32 and float(v.min()) >= 0.9 and float(v.max()) < 0.999 and float(v.std()) > 0.02
    n = host_values(TensorSpec("layer.gain", (4096,), "norm", init=("normal", 2.0, 0.25)), init)
    assert abs(float(n.mean()) - 2.0) < 0.02 and abs(float(n.std()) - 0.25) < 0.02
    c = host_values(TensorSpec("layer.one", (8,), "bias", init=("constant", -1.5)), init)
    assert torch.equal(c, torch.full((8,), -1.5))
    assert distribution(TensorSpec("w", (2, 2)), init) == (0, 0.0, 0.02)          # by role, as before


def test_slices_of_one_fused_tensor_in_different_types_are_refused_before_anything_is_allocated():
    specs = [TensorSpec(f"experts.{e}.down", (4, 4), into=("experts.down", (3, 4, 4), (e,))) for e in range(3)]
    held = {"experts.0.down": (torch.bfloat16, (4, 4)), "experts.1.down": (torch.float32, (4, 4)), "experts.2.down": (torch.bfloat16, (4, 4))}
    with pytest.raises(WeightsError, match="mixed types: the parts of experts.down are stored in different types") as err:
        check(specs, held, exact=False)
    assert sorted(n for n, _ in err.value.wrong_type) == sorted(held)
    check(specs, held, exact=True)          # the 32-bit path widens every slice to float32: no mix
    check(specs, {n: (torch.bfloat16, (4, 4)) for n in held}, exact=False)


def test_folder_loads_on_the_cpu_with_every_tensor_consumed_once():
    cfg = MiniMaxM3Config(**TINY_A)
    files = ModelFiles(model_folder("A"))
    specs = model_tensor_specs(cfg)
    assert sorted(s.name for s in specs) == sorted(files.names())
    tensors = load(specs, files, torch.device("cpu"), exact=False)
    assert tensors["model.layers.0.mlp.experts.gate_up_proj"].dtype == torch.bfloat16
    assert tensors["model.layers.0.mlp.gate.weight"].dtype == torch.float32
    assert tensors["model.layers.0.mlp.experts.gate_up_proj"].shape == (8, 64, 64)


def test_per_expert_tensor_names_are_an_alternative(tmp_path):
    """A file may hold experts.N.{gate,up,down}_proj.weight instead of the fused tensors; a mix of both is refused."""
    cfg = MiniMaxM3Config(**TINY_A)
    tensors = random_tensors(cfg, INIT_A)
    split = {}
    for name, t in tensors.items():
        if name.endswith("experts.gate_up_proj"):
            base = name[:-len("gate_up_proj")]
            for e in range(t.shape[0]):
                split[f"{base}{e}.gate_proj.weight"] = t[e, :32].clone()
                split[f"{base}{e}.up_proj.weight"] = t[e, 32:].clone()
        elif name.endswith("experts.down_proj"):
            base = name[:-len("down_proj")]
            for e in range(t.shape[0]):
                split[f"{base}{e}.down_proj.weight"] = t[e].clone()
        else:
            split[name] = t
    from llmx_amd.engine.model import BuiltModel
    from llmx_amd.models import assemble
    from llmx_amd.parts.base import BuildContext
    model = BuiltModel(assemble(cfg), BuildContext(torch.float32, torch.device("cpu"), 8))
    specs = model.tensor_specs(set(split))
    check(specs, {n: (t.dtype, tuple(t.shape)) for n, t in split.items()})
    # through the loader: every expert's tensors are copied from the host into their places in the fused tensors, so
    # what reaches the device is the fused pair alone (never the slices beside their fused copy)
    write_safetensors(tmp_path / "model.safetensors", split)
    files = ModelFiles(tmp_path)
    loaded = load(specs, files, torch.device("cpu"), exact=True)
    files.close()
    assert not any(".experts." in n and n.endswith("_proj.weight") for n in loaded)
    assert sum(t.numel() for t in loaded.values()) == sum(t.numel() for t in tensors.values())
    model.load(loaded)
    ffn = model.blocks[0].ffn
    assert torch.equal(ffn.w_gate_up, tensors["model.layers.0.mlp.experts.gate_up_proj"].float())
    assert torch.equal(ffn.w_down, tensors["model.layers.0.mlp.experts.down_proj"].float())
    mixed = dict(split)
    mixed["model.layers.0.mlp.experts.gate_up_proj"] = tensors["model.layers.0.mlp.experts.gate_up_proj"]
    with pytest.raises(ValueError, match="both fused and per-expert"):
        model.tensor_specs(set(mixed))


def test_random_weights_are_reproducible_per_tensor(tmp_path):
    init = RandomInit(seed=7, std=0.05, norm_std=0.1, bias_range=0.1)
    a = host_values(TensorSpec("model.layers.0.self_attn.q_proj.weight", (64, 64)), init)
    b = host_values(TensorSpec("model.layers.0.self_attn.q_proj.weight", (64, 64)), init)
    c = host_values(TensorSpec("model.layers.1.self_attn.q_proj.weight", (64, 64)), init)
    d = host_values(TensorSpec("model.layers.0.self_attn.q_proj.weight", (64, 64)), RandomInit(seed=8, std=0.05))
    assert torch.equal(a, b) and not torch.equal(a, c) and not torch.equal(a, d)
    assert abs(float(a.std()) - 0.05) < 5e-3 and abs(float(a.mean())) < 5e-3
    n = host_values(TensorSpec("x.weight", (4096,), "norm"), init)
    assert abs(float(n.mean()) - 1.0) < 1e-2 and abs(float(n.std()) - 0.1) < 1e-2
    bias = host_values(TensorSpec("x.bias", (4096,), "bias"), init)
    assert float(bias.min()) >= -0.1 and float(bias.max()) < 0.1 and float(bias.std()) > 0.05
    ones = host_values(TensorSpec("x.weight", (16,), "norm"), RandomInit(seed=0))
    assert torch.equal(ones, torch.ones(16))
    folder = write_random_model(tmp_path / "r", MiniMaxM3Config(**TINY_A), RandomInit(seed=0))
    again = write_random_model(tmp_path / "r2", MiniMaxM3Config(**TINY_A), RandomInit(seed=0))
    assert (folder / "model.safetensors").read_bytes() == (again / "model.safetensors").read_bytes()
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["MiniMaxM3ForCausalLM"]
