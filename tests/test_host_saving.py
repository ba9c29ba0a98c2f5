"""Saving and loading in the reference's formats, on the host.

Golden vector: `tests/golden/ref_nested_container.keras`, a `.keras` archive written by the
reference itself (keras/src/saving/test_data/pre_pr22362_nested_container.keras, Keras
3.15 + h5py).  The reference's own test of that file
(keras/src/saving/saving_lib_test.py:1306-1383) states what it holds: three bias-free
Dense(4) kernels filled with 0.1 * (i + 1), an output Dense(2) with kernel 0.5 and bias 0,
stored under `/layers/dense*` because the writer of that version did not walk nested
containers, and loading it must warn "Skipping nested container".
"""

import io
import json
import os
import struct
import warnings
import zipfile

import numpy as np
import pytest
import torch

import keras_amd as ka
from keras_amd import saving
from keras_amd.models import Model
from keras_amd.saving import h5min

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "ref_nested_container.keras")


def fixture_h5():
    with zipfile.ZipFile(FIXTURE) as zf:
        return zf.read("model.weights.h5")


def flatten(group, prefix=""):
    out = {}
    for name, node in group.items():
        path = f"{prefix}/{name}"
        if isinstance(node, h5min.Group):
            out[path] = dict(node.attrs)
            out.update(flatten(node, path))
        else:
            out[path] = node
    return out


# ---------------------------------------------------------------------------- the HDF5 subset


def test_reader_recovers_the_reference_file():
    flat = flatten(h5min.load(fixture_h5()))
    assert flat["/vars"] == {"name": "nested_dense_model"}
    for i, (path, name) in enumerate([("/layers/dense", "d_0"), ("/layers/dense_1", "d_1"),
                                      ("/layers/dense_2", "d_2")]):
        assert flat[path + "/vars"] == {"name": name}
        kernel = flat[path + "/vars/0"].value
        assert kernel.dtype == np.float32 and kernel.shape == (4, 4)
        np.testing.assert_allclose(kernel, np.full((4, 4), 0.1 * (i + 1), dtype="float32"), atol=1e-6)
        assert path + "/vars/1" not in flat  # use_bias=False
    assert flat["/layers/dense_3/vars"] == {"name": "dense"}
    np.testing.assert_allclose(flat["/layers/dense_3/vars/0"].value, np.full((4, 2), 0.5, dtype="float32"))
    np.testing.assert_array_equal(flat["/layers/dense_3/vars/1"].value, np.zeros((2,), dtype="float32"))
    assert set(p for p in flat if not p.count("/vars")) == {
        "/layers", "/layers/dense", "/layers/dense_1", "/layers/dense_2", "/layers/dense_3"}


def header_messages(data):
    """{object path: [(message type, body bytes)]} of every object in a file."""
    r = h5min._Reader(data)
    out = {}

    def walk(addr, path):
        msgs = r.messages(addr)
        out[path] = [(t, data[b:b + s]) for t, b, s in msgs if t not in (0x0, 0x10, 0x12)]
        for t, b, _ in msgs:
            if t == 0x11:
                btree, heap = struct.unpack_from("<QQ", data, b)
                for name, child in r.symbols(btree, heap, 0):
                    walk(child, f"{path}/{name}")

    walk(struct.unpack_from("<Q", data, 64)[0], "")
    return out


def test_writer_emits_the_messages_h5py_wrote():
    # re-serialize the reference's tree: every header message (dataspace, datatype, fill value,
    # layout, attribute) must come out byte for byte as h5py wrote it, addresses aside
    original = fixture_h5()
    rewritten = h5min.dump(h5min.load(original))
    a, b = header_messages(original), header_messages(rewritten)
    assert a.keys() == b.keys()
    checked = 0
    for path in a:
        ma, mb = dict(a[path]), dict(b[path])
        assert ma.keys() == mb.keys(), path
        for mtype in ma:
            x, y = ma[mtype], mb[mtype]
            if mtype == 0x11:      # symbol table: two addresses
                continue
            if mtype == 0x8:       # layout: version, class, size (not the data address)
                x, y = x[:2] + x[10:18], y[:2] + y[10:18]
            if mtype == 0xC:       # attribute: all but global-heap address and index
                x, y = x[:-12], y[:-12]
            assert x == y, (path, hex(mtype))
            checked += 1
    assert checked == 25
    # superblock: same versions, sizes, group K values and root entry layout
    assert original[:24] == rewritten[:24]
    assert flatten(h5min.load(rewritten)).keys() == flatten(h5min.load(original)).keys()


def test_rejects_what_is_outside_the_subset():
    with pytest.raises(h5min.H5FormatError, match="signature"):
        h5min.load(b"not an hdf5 file" * 10)
    data = bytearray(fixture_h5())
    data[8] = 2  # superblock version
    with pytest.raises(h5min.H5FormatError, match="superblock version 2"):
        h5min.load(bytes(data))
    with pytest.raises(h5min.H5FormatError):
        h5min.load(fixture_h5()[:4000])  # truncated


@pytest.mark.parametrize("count", [0, 1, 8, 9, 40, 300, 700])
def test_group_sizes_cross_node_boundaries(count):
    # 8 entries fill a symbol-table node, 256 a level-0 B-tree node: larger groups need more
    # of both; names must come back complete and datasets intact
    root = h5min.Group()
    g = root.require_group("layers")
    for i in range(count):
        g[f"dense_{i}"] = h5min.Dataset(np.full((3,), i, dtype=np.int32), {"dtype": "x" * (i % 5)})
    back = h5min.load(h5min.dump(root))["layers"]
    assert sorted(back) == sorted(f"dense_{i}" for i in range(count))
    for i in range(count):
        np.testing.assert_array_equal(back[f"dense_{i}"].value, np.full((3,), i, dtype=np.int32))
        assert back[f"dense_{i}"].attrs["dtype"] == "x" * (i % 5)


def test_btree_keys_are_ordered_heap_offsets():
    root = h5min.Group({f"n{i:03d}": h5min.Dataset(np.zeros(1, np.int8)) for i in range(100)})
    data = h5min.dump(root)
    btree, heap = struct.unpack_from("<QQ", data, 80)
    names_at = struct.unpack_from("<Q", data, heap + 24)[0]
    level, used = struct.unpack_from("<BH", data, btree + 5)
    assert level == 0 and used == 13  # 100 entries over ceil(100 / 8) nodes
    keys = [struct.unpack_from("<Q", data, btree + 24 + 16 * i)[0] for i in range(used + 1)]
    names = [data[names_at + k:data.index(b"\0", names_at + k)].decode() for k in keys]
    assert names[0] == "" and names[1:] == sorted(names[1:]) and names[-1] == "n099"
    for i in range(used):  # every node holds 4..8 symbols, all <= its right key
        child = struct.unpack_from("<Q", data, btree + 32 + 16 * i)[0]
        assert data[child:child + 4] == b"SNOD"
        n = struct.unpack_from("<H", data, child + 6)[0]
        assert 4 <= n <= 8


@pytest.mark.parametrize("dtype", ["int8", "uint8", "int32", "int64", "float16", "float32", "float64"])
def test_number_types_round_trip(dtype):
    rng = np.random.default_rng(0)
    arr = (rng.standard_normal((5, 7)) * 50).astype(dtype)
    root = h5min.Group({"a": h5min.Dataset(arr), "scalar": h5min.Dataset(np.array(3, dtype=dtype)),
                        "empty": h5min.Dataset(np.zeros((0, 4), dtype=dtype))})
    back = h5min.load(h5min.dump(root))
    assert back["a"].value.dtype == np.dtype(dtype)
    np.testing.assert_array_equal(back["a"].value, arr)
    assert back["scalar"].value.shape == () and back["scalar"].value == 3
    assert back["empty"].value.shape == (0, 4)


def test_int8_and_bfloat16_dataset_encodings_follow_the_format_specification():
    # No file in the reference tree holds an int8 or a bfloat16 dataset, so these two encodings
    # are pinned by what the HDF5 File Format Specification (version 3, IV.A.2.d "The Datatype
    # Message") fixes, field by field:
    #   byte 0      version (high nibble) = 1, class (low nibble): 0 fixed-point, 5 opaque
    #   bytes 1-3   class bit field
    #   bytes 4-7   element size
    #   then the class's properties
    # int8 = what `group[key] = int8 ndarray` makes h5py emit (H5T_STD_I8LE): class 0; bit 0 = 0
    # little-endian, bits 1-2 = 0 zero padding, bit 3 = 1 two's-complement signed; size 1;
    # properties: bit offset 0 (uint16), bit precision 8 (uint16).
    int8_message = bytes([0x10, 0x08, 0x00, 0x00, 0x01, 0x00, 0x00, 0x00, 0x00, 0x00, 0x08, 0x00])
    # bfloat16 = what `create_dataset(key, data=<ml_dtypes.bfloat16 array>)` asks for
    # (keras/src/saving/saving_lib.py:1469-1473): numpy sees a 2-byte void-kind dtype, which
    # h5py maps to H5T_OPAQUE of that size with no tag: class 5; bits 0-7 = length of the ASCII
    # tag = 0; size 2; no properties.  The value's meaning travels in the attribute
    # dtype = "bfloat16" (saving_lib.py:1455-1459 reads it back through that attribute).
    opaque2_message = bytes([0x15, 0x00, 0x00, 0x00, 0x02, 0x00, 0x00, 0x00])
    assert h5min._datatype_message(np.int8) == int8_message
    assert h5min._datatype_message(np.dtype("V2")) == opaque2_message
    # unsigned differs in the sign bit only
    assert h5min._datatype_message(np.uint8) == bytes([0x10, 0x00, 0, 0, 1, 0, 0, 0, 0, 0, 8, 0])

    rng = np.random.default_rng(3)
    q = rng.integers(-128, 128, size=(6, 10), dtype=np.int8)
    bf16_bits = rng.integers(0, 1 << 16, size=(4, 3), dtype=np.uint16)
    root = h5min.Group({"vars": h5min.Group({
        "0": h5min.Dataset(q),
        "1": h5min.Dataset(bf16_bits.view("V2"), attrs={"dtype": "bfloat16"})})})
    data = h5min.dump(root)
    # the messages sit in the datasets' (version 1) object headers: type 0x0003, their length
    # padded to 8, flags 1 (constant), three reserved bytes, then the body
    for body in (int8_message, opaque2_message):
        padded = body + b"\0" * (-len(body) % 8)
        assert struct.pack("<HHB3x", 0x0003, len(padded), 1) + padded in data
    # the int8 values lie in the file as they lie in memory (contiguous layout, row-major)
    assert q.tobytes() in data and bf16_bits.tobytes() in data
    # and the reader -- the code path the reference-written fixture pins for float32 datasets,
    # attributes and groups -- decodes both
    back = h5min.load(data)["vars"]
    assert back["0"].value.dtype == np.int8 and np.array_equal(back["0"].value, q)
    assert back["1"].value.dtype == np.dtype("V2")
    assert np.array_equal(back["1"].value.view(np.uint16), bf16_bits)
    assert back["1"].attrs["dtype"] == "bfloat16"
    # through the store: a bfloat16 tensor comes back as the same bits, an int8 tensor as int8
    t = torch.randn(5, 4).to(torch.bfloat16)
    buf = io.BytesIO()
    store = saving.H5Store(buf, mode="w")
    entry = store.make("layers/dense")
    entry["0"] = torch.from_numpy(q)
    entry["1"] = t
    store.close()
    for body in (int8_message, opaque2_message):
        padded = body + b"\0" * (-len(body) % 8)
        assert struct.pack("<HHB3x", 0x0003, len(padded), 1) + padded in buf.getvalue()
    rd = saving.H5Store(io.BytesIO(buf.getvalue()), mode="r").get("layers/dense")
    assert np.array_equal(np.asarray(rd["0"]), q) and np.asarray(rd["0"]).dtype == np.int8
    assert rd["1"].dtype == torch.bfloat16 and torch.equal(rd["1"].view(torch.int16), t.view(torch.int16))


# ---------------------------------------------------------------------------- the model walk


class NestedDenseModel(Model):
    """The model class of the reference's fixture (saving_lib_test.py:1326-1345)."""

    def __init__(self, num=3, **kwargs):
        super().__init__(**kwargs)
        self.num = num
        self.blocks = [(ka.layers.Dense(4, use_bias=False, name=f"d_{i}", device="cpu"),) for i in range(num)]
        self.out = ka.layers.Dense(2, device="cpu")
        for (d,) in self.blocks:
            d.build((2, 4))
        self.out.build((2, 4))

    def get_config(self):
        cfg = super().get_config()
        cfg["num"] = self.num
        return cfg


def test_loads_the_reference_archive_like_the_reference_does():
    model = NestedDenseModel(device="cpu")
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        model.load_weights(FIXTURE)
    assert sum("Skipping nested container" in str(w.message) for w in caught) == 3
    for i, (d,) in enumerate(model.blocks):
        np.testing.assert_allclose(d.kernel.numpy(), np.full((4, 4), 0.1 * (i + 1), dtype="float32"), atol=1e-6)
    np.testing.assert_allclose(model.out.kernel.numpy(), np.full((4, 2), 0.5, dtype="float32"), atol=1e-6)
    np.testing.assert_allclose(model.out.bias.value.numpy(), np.zeros((2,), dtype="float32"), atol=1e-6)


def test_walk_paths_and_names(tmp_path):
    # the layout the reference writes today: nested containers are walked, `layers` comes after
    # `blocks` and only adds what was not visited (its counter still advances: dense_3)
    model = NestedDenseModel(device="cpu")
    path = tmp_path / "m.weights.h5"
    model.save_weights(path)
    flat = flatten(h5min.load(path.read_bytes()))
    assert flat["/vars"] == {"name": "nested_dense_model"}
    assert flat["/blocks/container/dense/vars"] == {"name": "d_0"}
    assert flat["/blocks/container_1/dense/vars"] == {"name": "d_1"}
    assert flat["/blocks/container_2/dense/vars"] == {"name": "d_2"}
    assert flat["/layers/dense_3/vars"] == {"name": "dense"}
    assert flat["/layers/dense_3/vars/1"].value.shape == (2,)
    assert "/layers/dense" not in flat and "/out" not in flat
    with pytest.raises(ValueError, match=r"must end in `.weights.h5`"):
        model.save_weights(tmp_path / "m.h5")


def test_missing_variables_are_reported(tmp_path):
    small = NestedDenseModel(num=1, device="cpu")
    path = tmp_path / "small.weights.h5"
    small.save_weights(path)
    big = NestedDenseModel(num=3, device="cpu")
    # d_1 meets the small model's output kernel at layers/dense_1 (wrong shape), d_2 and the
    # output layer meet nothing
    with pytest.raises(ValueError, match="A total of 3 objects could not be loaded"):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            big.load_weights(path)


# ---------------------------------------------------------------------------- quantized layers


class QuantizedStack(Model):
    def __init__(self, dtype="float32", **kwargs):
        super().__init__(dtype=dtype, **kwargs)
        kw = dict(dtype=dtype, device="cpu")
        self.embed = ka.layers.ReversibleEmbedding(64, 32, tie_weights=False, **kw)
        self.tok = ka.layers.Embedding(48, 32, **kw)
        self.proj = ka.layers.EinsumDense("abc,cde->abde", output_shape=(None, 4, 8), bias_axes="e", **kw)
        self.ffn = [ka.layers.Dense(64, activation="relu", **kw), ka.layers.Dense(32, use_bias=False, **kw)]
        self.embed.build()
        self.tok.build()
        self.proj.build((2, 3, 32))
        self.ffn[0].build((2, 32))
        self.ffn[1].build((2, 64))

    def get_config(self):
        return {"name": self.name, "dtype": self.dtype_policy.name}


def randomize(model):
    g = torch.Generator().manual_seed(3)
    for layer in model._flatten_layers():
        for v in layer._variables:
            t = v.value
            if t.dtype == torch.int8:
                v.assign(torch.randint(-128, 128, t.shape, generator=g, dtype=torch.int8))
            elif "g_idx" not in v.name:
                v.assign((torch.rand(t.shape, generator=g) + 0.5).to(t.dtype))


def variables_of(model):
    out = {}
    for i, layer in enumerate(model._flatten_layers()):
        for v in layer._variables:
            out[(i, v.name)] = v.value
    return out


@pytest.mark.parametrize("dtype", ["float32", "mixed_bfloat16", "bfloat16"])
@pytest.mark.parametrize("mode", [None, "int8", "int4"])
def test_quantized_model_round_trip(tmp_path, dtype, mode):
    torch.manual_seed(0)
    if mode == "int4":
        # packing int4 runs on the device only: build the layers under the quantized policy
        # (as loading a saved model does) and fill their variables
        model = QuantizedStack(dtype=f"int4/16_from_{dtype}", name="stack", device="cpu")
        randomize(model)
    else:
        model = QuantizedStack(dtype=dtype, name="stack", device="cpu")
        if mode is not None:
            report = model.quantize(mode)
            assert report.num_quantized == 5
    path = tmp_path / "stack.keras"
    model.save(path)

    with zipfile.ZipFile(path) as zf:
        assert sorted(zf.namelist()) == ["config.json", "metadata.json", "model.weights.h5"]
        meta = json.loads(zf.read("metadata.json"))
        assert set(meta) == {"keras_version", "date_saved"}
        cfg = json.loads(zf.read("config.json"))
        assert cfg["class_name"] == "QuantizedStack" and cfg["config"]["name"] == "stack"
        flat = flatten(h5min.load(zf.read("model.weights.h5")))
    # positional keys follow variable_serialization_spec (dense.py:486-541): kernel, bias,
    # kernel_scale, kernel_zero, g_idx with absent entries skipped
    expected_keys = {None: 2, "int8": 3, "int4": 5}[mode]
    dense0 = [p for p in flat if p.startswith("/ffn/dense/vars/")]
    assert len(dense0) == expected_keys
    dense1 = [p for p in flat if p.startswith("/ffn/dense_1/vars/")]
    assert len(dense1) == expected_keys - 1  # no bias
    if mode is not None:
        assert flat["/ffn/dense/vars/0"].value.dtype == np.int8
    # bfloat16 variables: 2-byte opaque elements tagged dtype="bfloat16" (saving_lib.py:1459-1465)
    scale = flat["/ffn/dense/vars/1"]
    if dtype == "bfloat16":
        assert scale.value.dtype == np.dtype("V2") and scale.attrs == {"dtype": "bfloat16"}
    else:
        assert scale.value.dtype == np.float32 and scale.attrs == {}

    fresh = QuantizedStack(dtype=model.dtype_policy.name, name="other", device="cpu")
    if mode == "int8":
        fresh.quantize(mode)
    before = variables_of(fresh)
    fresh.load_weights(path)
    want, got = variables_of(model), variables_of(fresh)
    assert want.keys() == got.keys() and len(want) >= 8
    changed = 0
    for name in want:
        assert got[name].dtype == want[name].dtype and torch.equal(got[name], want[name]), name
        changed += not torch.equal(before[name], got[name])
    assert changed >= 5  # the load did replace freshly initialised values


def test_load_model_rebuilds_quantized_layers(tmp_path):
    torch.manual_seed(1)
    # built under the quantized policy (packing on quantize() needs the device)
    layer = ka.layers.Dense(16, activation="relu", dtype="int4/16_from_mixed_bfloat16", name="head",
                            device="cpu", quantization_config=ka.Int4QuantizationConfig(block_size=16))
    layer.build((4, 32))
    holder = Model(device="cpu")
    holder.head = layer
    randomize(holder)
    path = tmp_path / "head.keras"
    saving.save_model(layer, path)
    with zipfile.ZipFile(path) as zf:
        cfg = json.loads(zf.read("config.json"))
    assert cfg["module"] == "keras.layers" and cfg["class_name"] == "Dense" and cfg["registered_name"] is None
    assert cfg["config"]["dtype"] == "int4/16_from_mixed_bfloat16"
    assert cfg["config"]["quantization_config"]["class_name"] == "Int4QuantizationConfig"
    assert cfg["build_config"] == {"input_shape": [4, 32]}
    back = saving.load_model(path, device="cpu")
    assert type(back) is ka.layers.Dense and back.quantization_mode == "int4" and back.name == "head"
    assert back._int4_block_size == 16
    for a, b in zip(layer._variables, back._variables):
        assert a.name == b.name and torch.equal(a.value, b.value)
    with pytest.raises(TypeError, match="Could not locate class 'QuantizedStack'"):
        model = QuantizedStack(device="cpu")
        model.save(tmp_path / "m.keras")
        saving.load_model(tmp_path / "m.keras")
    again = saving.load_model(tmp_path / "m.keras", custom_objects={"QuantizedStack": QuantizedStack})
    assert isinstance(again, QuantizedStack)


def test_store_semantics():
    buf = io.BytesIO()
    store = saving.H5Store(buf, mode="w")
    with pytest.raises(ValueError, match="only allowed in write mode"):
        saving.H5Store(io.BytesIO(h5min.dump(h5min.Group())), mode="r").make("x")
    store.make("layers/unused")  # no variable written: no group appears
    entry = store.make("layers/dense")
    entry["0"] = torch.arange(6, dtype=torch.int8).reshape(2, 3)
    entry["1"] = torch.tensor([1.5, -2.0], dtype=torch.bfloat16)
    store.make("", metadata={"name": "root"})
    store.close()
    back = saving.H5Store(io.BytesIO(buf.getvalue()), mode="r")
    assert not back.has_path("layers/unused") and back.has_path("layers/dense")
    entry = back.get("layers/dense")
    assert list(entry.keys()) == ["0", "1"] and len(entry) == 2 and "0" in entry
    assert entry["0"].dtype == np.int8 and entry["0"].tolist() == [[0, 1, 2], [3, 4, 5]]
    assert entry["1"].dtype == torch.bfloat16 and entry["1"].tolist() == [1.5, -2.0]
    assert len(back.get("layers/missing")) == 0
    assert back.root["vars"].attrs == {"name": "root"}
