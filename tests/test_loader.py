"""No-GPU checks of the loader glue: the library's safetensors reader against files written here with
Python's json module (and read back by the `safetensors` package as an independent witness), LoadLinear's
per-weight decisions (go/model/linear.go:42-84) and the 1-bit -> 2-bit widening
(go/model/quant/mlxaffine/repack.go:27-62)."""
import json
import os
import struct

import numpy as np
import pytest

import fixtures as F


def write_safetensors(path, tensors, metadata=None, extra_keys=False):
    """tensors: {name: (dtype string, shape, bytes-like)} -> a safetensors file."""
    header, blobs, off = {}, [], 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, (dtype, shape, data) in tensors.items():
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1).tobytes()
        entry = {"dtype": dtype, "shape": list(shape), "data_offsets": [off, off + len(raw)]}
        if extra_keys:
            entry = {"future": {"nested": [1, 2.5, "x", None, True]}, **entry, "also": "ignored"}
        header[name] = entry
        blobs.append(raw)
        off += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def affine_entry(prefix, N, K, bits, gs, seed, experts=0):
    rows = N * max(experts, 1)
    if 32 % bits == 0:
        w, s, b = F.synthetic_affine(rows, K, bits, gs, seed=seed)
    else:
        rng = np.random.default_rng(seed)
        w = F.pack_codes(rng.integers(0, 1 << bits, size=(rows, K)), bits)
        s = F.f32_to_bf16_bits(rng.normal(0, 0.02, (rows, K // gs)).astype(np.float32))
        b = F.f32_to_bf16_bits(rng.normal(0, 0.05, (rows, K // gs)).astype(np.float32))
    lead = [experts, N] if experts else [N]
    return {prefix + ".weight": ("U32", lead + [K * bits // 32], w), prefix + ".scales": ("BF16", lead + [K // gs], s),
            prefix + ".biases": ("BF16", lead + [K // gs], b)}, (w, s, b)


@pytest.fixture()
def model_file(tmp_path):
    import aq_mi355
    tensors, want = {}, {}
    for name, (N, K, bits, gs, experts) in {"layers.0.q_proj": (24, 256, 4, 64, 0), "layers.0.k_proj": (8, 256, 8, 64, 0),
                                            "layers.0.v_proj": (8, 256, 6, 32, 0), "layers.0.o_proj": (16, 128, 5, 64, 0),
                                            "layers.0.experts.gate_proj": (12, 128, 4, 64, 3),
                                            "layers.0.experts.up_proj": (12, 128, 4, 64, 3)}.items():
        t, w = affine_entry(name, N, K, bits, gs, seed=len(tensors) + 1, experts=experts)
        tensors.update(t)
        want[name] = (w, (N, K, bits, gs, experts))
    dense = F.f32_to_bf16_bits(np.random.default_rng(3).normal(0, 1, (10, 64)).astype(np.float32))
    tensors["layers.0.dense_proj.weight"] = ("BF16", [10, 64], dense)
    tensors["layers.0.dense_proj.bias"] = ("BF16", [10], dense[0, :10])
    tensors['odd "name"\\with\u00e9'] = ("U8", [3], np.array([1, 2, 3], np.uint8))
    tensors["empty"] = ("F32", [0, 4], np.zeros(0, np.float32))
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, tensors, metadata={"format": "mlx", "note": "caf\u00e9"}, extra_keys=True)
    f = aq_mi355.SafetensorsFile(path)
    yield f, tensors, want, path
    f.close()


def test_reader_agrees_with_the_safetensors_package(model_file):
    safetensors = pytest.importorskip("safetensors")
    f, tensors, _, path = model_file
    assert f.names() == sorted(tensors)
    with safetensors.safe_open(path, framework="np") as ref:      # the file is one the reference library accepts
        assert sorted(ref.keys()) == sorted(tensors)
        for name in ("layers.0.q_proj.weight", "odd \"name\"\\with\u00e9", "empty"):
            assert list(ref.get_slice(name).get_shape()) == list(tensors[name][1])
        assert np.array_equal(ref.get_tensor("layers.0.q_proj.weight"), tensors["layers.0.q_proj.weight"][2])
    for name, (dtype, shape, data) in tensors.items():
        d, s, view = f.tensor(name)
        assert (d, s) == (dtype, list(shape))
        assert np.array_equal(view, np.ascontiguousarray(data).view(np.uint8).reshape(-1))


def test_load_linear_decides_per_weight(model_file):
    """go/model/linear.go:42-84: geometry from the shapes; no scales -> dense; no weight -> nil."""
    f, _, want, _ = model_file
    for name, ((w, s, b), (N, K, bits, gs, experts)) in want.items():
        lin = f.load_linear(name, K)
        assert lin is not None and lin.quantised == 1
        assert (lin.group_size, lin.bits, lin.in_dim) == (gs, bits, K)
        assert lin.out_dim == (experts or N)                      # firstDim of the weight, as the Go loader reads it
        assert (lin.experts, lin.expert_rows) == (experts, N)
        assert np.array_equal(lin.view("weight"), w.view(np.uint8).reshape(-1))
        assert np.array_equal(lin.view("scales"), s.view(np.uint8).reshape(-1))
        assert np.array_equal(lin.view("biases"), b.view(np.uint8).reshape(-1))
        assert lin.view("bias") is None
    dense = f.load_linear("layers.0.dense_proj", 64)
    assert dense.quantised == 0 and dense.scales is None and (dense.group_size, dense.bits) == (0, 0)
    assert dense.out_dim == 10 and dense.bias_len == 20
    assert f.load_linear("layers.0.missing_proj", 64) is None


def test_one_bit_pack_is_widened_and_written_back(tmp_path, orc):
    """go/model/linear.go:62-80 + repack.go:27-62, against the oracle's restatement; dequant is unchanged."""
    import aq_mi355
    N, K, gs = 6, 128, 64
    rng = np.random.default_rng(11)
    w1 = rng.integers(0, 1 << 32, size=(N, K // 32), dtype=np.uint64).astype(np.uint32)
    s = F.f32_to_bf16_bits(rng.normal(0, 0.1, (N, K // gs)).astype(np.float32))
    b = F.f32_to_bf16_bits(rng.normal(0, 0.1, (N, K // gs)).astype(np.float32))
    path = str(tmp_path / "bonsai.safetensors")
    write_safetensors(path, {"p.weight": ("U32", [N, K // 32], w1), "p.scales": ("BF16", [N, K // gs], s),
                             "p.biases": ("BF16", [N, K // gs], b)})
    f = aq_mi355.SafetensorsFile(path)
    lin = f.load_linear("p", K)
    assert (lin.bits, lin.group_size, lin.weight_len) == (2, gs, N * K // 4)
    want = orc.repack_b1_to_b2(w1, N, K)
    assert np.array_equal(lin.view("weight"), want)
    assert np.array_equal(orc.dequantize(lin.view("weight"), s, b, N, K, 2, gs), orc.dequantize(w1, s, b, N, K, 1, gs))
    # the widened weight replaced the tensor: a second (tied) read sees 2-bit codes and the same buffer
    d, shape, view = f.tensor("p.weight")
    assert shape == [N, K // 16] and np.array_equal(view, want)
    again = f.load_linear("p", K)
    assert again.bits == 2 and again.weight == lin.weight
    # the bare repack door, and its rejections
    lib = aq_mi355.load()
    out = np.zeros(N * K // 4, np.uint8)
    u8 = w1.view(np.uint8).reshape(-1)
    assert lib.aqh_repack_b1_to_b2(u8.ctypes.data, u8.size, s.nbytes, b.nbytes, N, K, gs, out.ctypes.data, out.size) == 0
    assert np.array_equal(out, want)
    assert lib.aqh_repack_b1_to_b2(u8.ctypes.data, u8.size - 4, s.nbytes, b.nbytes, N, K, gs, out.ctypes.data, out.size) != 0
    assert lib.aqh_repack_b1_to_b2(u8.ctypes.data, u8.size, s.nbytes, b.nbytes, N, 48, 16, out.ctypes.data, out.size) != 0
    f.close()


@pytest.mark.parametrize("case", ["short", "header_size", "not_json", "missing_field", "offsets_reversed", "offsets_outside",
                                  "length_mismatch", "negative_offset", "shape_product_wraps", "no_file"])
def test_malformed_files_are_rejected(tmp_path, case):
    import aq_mi355
    path = str(tmp_path / (case + ".safetensors"))
    good = {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}
    def emit(header, payload=b"\x01\x02\x03\x04", size=None):
        hj = header if isinstance(header, bytes) else json.dumps(header).encode()
        with open(path, "wb") as f:
            f.write(struct.pack("<Q", len(hj) if size is None else size) + hj + payload)
    if case == "short":
        open(path, "wb").write(b"\x01\x02\x03")
    elif case == "header_size":
        emit({"t": good}, size=1 << 40)
    elif case == "not_json":
        emit(b'{"t": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]')
    elif case == "missing_field":
        emit({"t": {"dtype": "U8", "shape": [4]}})
    elif case == "offsets_reversed":
        emit({"t": {**good, "data_offsets": [4, 0]}})
    elif case == "offsets_outside":
        emit({"t": {**good, "shape": [8], "data_offsets": [0, 8]}})
    elif case == "length_mismatch":
        emit({"t": {**good, "dtype": "U32"}})
    elif case == "negative_offset":
        emit({"t": {**good, "data_offsets": [-1, 3]}})
    elif case == "shape_product_wraps":     # 2^16 * 2^16 * 2^16 * 2^16 * 4 wraps to 4 in 64 bits
        emit({"t": {**good, "shape": [65536, 65536, 65536, 65536, 4]}})
    with pytest.raises(aq_mi355.AqError):
        aq_mi355.SafetensorsFile(path)
    if case == "no_file":
        return
    emit({"t": good})                       # the same framing with a sound header loads
    f = aq_mi355.SafetensorsFile(path)
    assert f.tensor("t")[2].tolist() == [1, 2, 3, 4]
    f.close()
    emit(b'{"a\\ud83d\\ude00": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}}')
    f = aq_mi355.SafetensorsFile(path)      # escapes decode one by one, as in the reference: two three-byte sequences
    assert f.tensor(b"a\xed\xa0\xbd\xed\xb8\x80")[2].tolist() == [1, 2, 3, 4]
    with pytest.raises(aq_mi355.AqError) as e:
        f.tensor("absent")
    assert e.value.code == aq_mi355.AQ_ERR_INDEX
    f.close()
