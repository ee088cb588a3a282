"""Weight import: the safetensors validation of the reference host restated
(crates/forja-host/src/weights.rs:395-465 and its tests :536-646), and a checkpoint in MLX naming
loaded into one read-only buffer whose tensors feed the quantised ops.  The tensors of the
checkpoint are the ones derived from the reference's tiny fixture (tests/golden)."""
import json
import os
import struct

import numpy as np
import pytest

from forja_amd.core import BackendError, CommandList, DType, Op
from forja_amd.weights import ImportedWeights, SafetensorsFile, WeightError, import_safetensors
from tests.helpers import to_f32, upload, upload_raw

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def write_file(path, header, data=b"", pad=False):
    text = header if isinstance(header, (bytes, str)) else json.dumps(header)
    text = text.encode() if isinstance(text, str) else text
    if pad:
        text += b" " * (-len(text) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(text)) + text + data)
    return str(path)


def entry(dtype, shape, start, end):
    return {"dtype": dtype, "shape": shape, "data_offsets": [start, end]}


def test_parses_supported_tensor_metadata(tmp_path):
    header = {"__metadata__": {"format": "pt"}, "b": entry("BF16", [2, 3], 8, 20),
              "a": entry("U32", [2], 0, 8), "c": entry("F32", [], 20, 24), "d": entry("F16", [0, 5], 24, 24)}
    file = SafetensorsFile(write_file(tmp_path / "m.safetensors", header, bytes(24)))
    assert [t.name for t in file.tensors] == ["a", "b", "c", "d"]          # by offset
    assert file.tensors[1].dtype == DType.BF16 and file.tensors[1].shape == (2, 3)
    assert file.tensors[2].shape == () and file.data_len == 24


@pytest.mark.parametrize("header,data,kind", [
    ({"a": entry("F32", [4], 0, 16)}, bytes(8), "Truncated"),                       # data cut short
    ({"a": entry("F32", [2], 0, 8), "b": entry("F32", [2], 4, 12)}, bytes(12), "OverlappingRanges"),
    ({"a": entry("F32", [2], 16, 24)}, bytes(16), "Truncated"),                     # past the end
    ({"a": entry("I64", [1], 0, 8)}, bytes(8), "UnsupportedDtype"),
    ({"a": entry("F32", [3], 0, 8)}, bytes(8), "InvalidRange"),                     # length != shape
    ({"a": entry("F32", [2], 8, 0)}, bytes(8), "InvalidRange"),
    ({"a": {"dtype": "F32", "shape": [2]}}, bytes(8), "InvalidHeader"),
    ({"a": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 8]}}, bytes(8), "InvalidHeader"),
    ('{"a": {"dtype":"F32","shape":[1],"data_offsets":[0,4]}, "a": {"dtype":"F32","shape":[1],"data_offsets":[4,8]}}',
     bytes(8), "InvalidHeader"),                                                    # duplicate name
    ("[" * 100000, b"", "InvalidHeader"),                                           # deep nesting
    ("[1, 2]", b"", "InvalidHeader"),
])
def test_refuses_what_the_reference_refuses(tmp_path, header, data, kind):
    with pytest.raises(WeightError) as info:
        SafetensorsFile(write_file(tmp_path / "m.safetensors", header, data))
    assert info.value.kind == kind


def test_refuses_oversized_headers_before_reading_them_and_short_files(tmp_path):
    path = tmp_path / "big.safetensors"
    path.write_bytes(struct.pack("<Q", 100 * 1024 * 1024 + 1))
    with pytest.raises(WeightError) as info:
        SafetensorsFile(str(path))
    assert info.value.kind == "HeaderTooLarge"
    path.write_bytes(b"\x01\x02")
    with pytest.raises(WeightError) as info:
        SafetensorsFile(str(path))
    assert info.value.kind == "Truncated"
    with pytest.raises(WeightError) as info:
        SafetensorsFile(str(tmp_path))
    assert info.value.kind == "NotRegularFile"


def test_offsets_are_relative_to_the_data_region(tmp_path):
    header = {"x": entry("BF16", [1], 2, 4), "w": entry("U32", [1], 4, 8)}
    file = SafetensorsFile(write_file(tmp_path / "m.safetensors", header, bytes(8), pad=True))
    assert file.data_start % 8 == 0
    by_name = {t.name: t for t in file.tensors}
    assert by_name["x"].is_dtype_aligned and by_name["w"].is_dtype_aligned
    odd = SafetensorsFile(write_file(tmp_path / "o.safetensors", {"w": entry("U32", [1], 2, 6)}, bytes(6)))
    assert not odd.tensors[0].is_dtype_aligned


def tiny_checkpoint(tmp_path):
    """The golden tensors under MLX names, with a stacked expert triple beside them."""
    z = np.load(os.path.join(GOLDEN, "tiny_qwen_mlx4.npz"))
    rng = np.random.default_rng(5)
    experts = {"weight": rng.integers(0, 2 ** 32, (3, 16, 8), dtype=np.uint64).astype(np.uint32),
               "scales": (rng.integers(0x3c00, 0x3c80, (3, 16, 1))).astype(np.uint16),
               "biases": (rng.integers(0xbc00, 0xbc80, (3, 16, 1))).astype(np.uint16)}
    arrays = {}
    for prefix, key in (("language_model.lm_head", "lm_head"), ("language_model.model.embed_tokens", "embed")):
        arrays[prefix + ".weight"] = ("U32", z[key + "_packed"])
        arrays[prefix + ".scales"] = ("BF16", z[key + "_scales_bf16"])
        arrays[prefix + ".biases"] = ("BF16", z[key + "_biases_bf16"])
    for part, array in experts.items():
        arrays["language_model.model.layers.0.mlp.switch_mlp.gate_proj." + part] = \
            ("U32" if part == "weight" else "BF16", array)
    header, data = {"__metadata__": {"format": "mlx"}}, b""
    for name, (dtype, array) in arrays.items():
        raw = np.ascontiguousarray(array).tobytes()
        header[name] = entry(dtype, list(array.shape), len(data), len(data) + len(raw))
        data += raw
    return write_file(tmp_path / "model.safetensors", header, data, pad=True), z, experts


def check_checkpoint(backend, tmp_path):
    path, z, experts = tiny_checkpoint(tmp_path)
    weights = import_safetensors(backend, path)
    assert isinstance(weights, ImportedWeights) and len(weights.names()) == 9
    embed = weights.quantised("language_model.model.embed_tokens")
    head = weights.quantised("language_model.lm_head")
    assert embed[0].buffer == head[0].buffer == head[2].buffer          # one allocation
    assert backend.read(head[0]) == z["lm_head_packed"].tobytes()       # bytes as in the file
    with pytest.raises(WeightError):
        weights.tensor("language_model.lm_head.weight", (33, 9))
    with pytest.raises(KeyError):
        weights.tensor("language_model.lm_head.missing")
    ids = upload_raw(backend, z["prompt_token_ids"], DType.U32, (3,))
    rows = backend.alloc(DType.BF16, (3, 64))
    hidden = upload(backend, z["final_hidden_last"].reshape(1, 64), DType.F32)
    logits, token = backend.alloc(DType.F32, (1, 33)), backend.alloc(DType.U32, (1,))
    stacked = weights.quantised("language_model.model.layers.0.mlp.switch_mlp.gate_proj")
    assert stacked[0].shape == (3, 16, 8)
    x = upload(backend, np.linspace(-1, 1, 2 * 64).reshape(2, 64), DType.BF16)
    routes = upload_raw(backend, np.array([[2, 0], [1, 1]], dtype=np.uint32), DType.U32, (2, 2))
    routed = backend.alloc(DType.BF16, (2, 2, 16))
    commands = CommandList()
    commands.dispatch(Op.quant_embed(4, 64), [*embed, ids], rows)
    commands.dispatch(Op.quant_matmul(4, 64), [hidden, *head], logits)
    commands.dispatch(Op.argmax(), [logits], token)
    commands.dispatch(Op.gather_quant_matmul(4, 64), [x, *stacked, routes], routed)
    backend.submit(commands).wait()
    assert np.array_equal(to_f32(backend.read(rows), DType.BF16), z["hidden_state_0"].ravel())
    actual = to_f32(backend.read(logits), DType.F32)
    assert np.linalg.norm(actual - z["prompt_last_logits"]) / np.linalg.norm(z["prompt_last_logits"]) < 5e-3
    assert np.frombuffer(backend.read(token), np.uint32)[0] == z["first_greedy_token"][0]
    # imported weights are read-only
    commands = CommandList()
    commands.dispatch(Op.copy(), [ids], head[0].narrow(0, 0, 1).reshape((8,)).narrow(0, 0, 3))
    with pytest.raises(BackendError):
        backend.submit(commands).wait()
    return to_f32(backend.read(routed), DType.BF16)


def test_checkpoint_in_mlx_naming_feeds_the_quantised_ops_on_the_oracle(cpu, tmp_path):
    check_checkpoint(cpu, tmp_path)


@pytest.mark.gpu
def test_checkpoint_in_mlx_naming_feeds_the_quantised_ops_on_the_device(cpu, hip, tmp_path):
    device = check_checkpoint(hip, tmp_path)
    reference = check_checkpoint(cpu, tmp_path)
    assert np.allclose(device, reference, rtol=1e-2, atol=1e-2)
