"""Saving and loading quantized layers and models in the reference's file formats.

What is restated of keras/src/saving/saving_lib.py:
  * the variable store of a weights file, `H5IOStore` (:1289-1483): one HDF5 group
    `<inner_path>/vars` per saveable, datasets `"0", "1", ...` in the order of the layer's
    `variable_serialization_spec`, attribute `name` on the group, attribute
    `dtype = "bfloat16"` on bfloat16 datasets;
  * the walk over a model, `_save_state` / `_load_state` / `_walk_saveable` and the container
    naming of `_save_container_state` (:737-1098): children in sorted attribute order,
    private attributes last, list / tuple / dict members addressed by the snake-cased class
    name with a counter (`dense`, `dense_1`, ...), nested containers as `container`,
    `container_1`, ...;
  * `save_weights` / `load_weights` on `*.weights.h5` (:578-700) and the `.keras` archive:
    a zip of `config.json`, `metadata.json` and `model.weights.h5` (:75-260).
The HDF5 bytes come from `h5min` (no `h5py`).
"""

import datetime
import io
import json
import zipfile

import numpy as np
import torch

from keras_amd.layers.layer import Layer, Variable, _snake_case
from keras_amd.saving import h5min

_CONFIG_FILENAME = "config.json"
_METADATA_FILENAME = "metadata.json"
_VARS_FNAME_H5 = "model.weights.h5"
KERAS_VERSION = "3.16.0"  # the reference version whose formats are written


def to_snake_case(name):
    """keras/src/utils/naming.py:to_snake_case."""
    return _snake_case(name)


def _to_numpy(value):
    """-> (numpy array, is_bfloat16).  bfloat16 has no numpy dtype: its 16-bit patterns
    travel as 2-byte opaque elements, which is also what h5py makes of such an array."""
    if isinstance(value, Variable):
        value = value.value
    if isinstance(value, torch.Tensor):
        t = value.detach().cpu().contiguous()
        if t.dtype == torch.bfloat16:
            return t.view(torch.int16).numpy().view("V2"), True
        return t.numpy(), False
    return np.asarray(value), False


class H5Store:
    """`H5IOStore` over `h5min`: `make(path)` / `get(path)` select a saveable's `vars` group,
    item access reads and writes its datasets.  Write mode builds the tree in memory and
    `close()` emits the file (or the archive member)."""

    def __init__(self, path_or_io, archive=None, mode="r"):
        if mode not in ("w", "r"):
            raise ValueError(f"`mode` should be either 'w' or 'r'. Received: {mode}")
        self.path_or_io = path_or_io
        self.archive = archive
        self.mode = mode
        if mode == "w":
            self.root = h5min.Group()
        elif archive is not None:
            self.root = h5min.load(archive.read(str(path_or_io)))
        elif isinstance(path_or_io, io.BytesIO):
            self.root = h5min.load(path_or_io.getvalue())
        else:
            with open(path_or_io, "rb") as f:
                self.root = h5min.load(f.read())
        self._entry_path = None
        self._entry = {}
        self._entry_ready = False

    # -- entry selection ---------------------------------------------------------------
    def make(self, path, metadata=None):
        if self.mode != "w":
            raise ValueError("`make` is only allowed in write mode.")
        if not isinstance(metadata, (dict, type(None))):
            raise ValueError(f"`metadata` should be a dict or `None`. Received: {metadata}")
        self._entry_path = path
        if metadata:
            self._create_entry(path, metadata)
        else:
            # the group appears with the first variable: unused stores leave no empty groups
            self._entry, self._entry_ready = {}, False
        return self

    def get(self, path):
        if self.mode != "r":
            raise ValueError("`get` is only allowed in read mode.")
        self._entry_path, self._entry, self._entry_ready = path, {}, True
        node = self.root.lookup(path) if path else self.root
        if isinstance(node, h5min.Group) and isinstance(node.get("vars"), h5min.Group):
            self._entry = node["vars"]
        return self

    def has_path(self, path):
        return self.root.lookup(path) is not None

    def _create_entry(self, path, metadata=None):
        parent = self.root.require_group(path) if path else self.root
        if "vars" in parent:
            raise ValueError(f"Unable to create group (name already exists): {path}/vars")
        self._entry = parent["vars"] = h5min.Group()
        for k, v in (metadata or {}).items():
            self._entry.attrs[k] = v
        self._entry_ready = True

    def close(self):
        if self.mode != "w":
            return
        data = h5min.dump(self.root)
        if self.archive is not None:
            self.archive.writestr(str(self.path_or_io), data)
        elif isinstance(self.path_or_io, io.BytesIO):
            self.path_or_io.write(data)
        else:
            with open(self.path_or_io, "wb") as f:
                f.write(data)

    # -- the selected entry ---------------------------------------------------------------
    def __len__(self):
        return len(self._entry)

    def keys(self):
        return self._entry.keys()

    def __contains__(self, key):
        return key in self._entry

    def __getitem__(self, key):
        ds = self._entry[key]
        if not isinstance(ds, h5min.Dataset):
            raise KeyError(f"'{key}' is not a dataset")
        if ds.attrs.get("dtype") == "bfloat16":
            if ds.value.dtype.itemsize != 2:
                raise ValueError(f"dataset '{key}' is tagged bfloat16 but holds {ds.value.dtype}")
            bits = np.ascontiguousarray(ds.value).view(np.int16)
            return torch.from_numpy(bits.copy()).view(torch.bfloat16)
        return ds.value

    def __setitem__(self, key, value):
        if self.mode != "w":
            raise ValueError("Setting a value is only allowed in write mode.")
        if not self._entry_ready:
            self._create_entry(self._entry_path)
        arr, is_bf16 = _to_numpy(value)
        self._entry[key] = h5min.Dataset(arr, {"dtype": "bfloat16"} if is_bf16 else None)


# ------------------------------------------------------------------------------ the walk

_SKIP_ATTRS = None


def _attr_skipset():
    """Attributes every layer has: not part of a model's structure (`get_attr_skipset`,
    saving_lib.py:1913-1960, takes `dir()` of a bare instance in the same way)."""
    global _SKIP_ATTRS
    if _SKIP_ATTRS is None:
        _SKIP_ATTRS = set(dir(Layer(device="cpu"))) | {"_self_unconditional_dependency_names"}
    return _SKIP_ATTRS


def _name_key(name):
    return f"~{name}" if name.startswith("_") else name  # private attributes are visited last


def _walk(saveable):
    skip = _attr_skipset()
    for attr in sorted(dir(saveable), key=_name_key):
        if attr.startswith("__") or attr in skip:
            continue
        try:
            child = getattr(saveable, attr)
        except Exception:
            continue
        yield attr, child


def _unique_name(name, used):
    if name in used:
        used[name] += 1
        return f"{name}_{used[name]}"
    used[name] = 0
    return name


def _save_state(saveable, store, path="", visited=None):
    """`_save_state` (saving_lib.py:768-830)."""
    visited = set() if visited is None else visited
    if id(saveable) in visited:
        return
    if hasattr(saveable, "save_own_variables"):
        metadata = {"name": saveable.name} if isinstance(getattr(saveable, "name", None), str) else None
        saveable.save_own_variables(store.make(path, metadata=metadata))
    visited.add(id(saveable))
    for attr, child in _walk(saveable):
        sub = f"{path}/{attr}" if path else attr
        if isinstance(child, Layer):
            _save_state(child, store, sub, visited)
        elif isinstance(child, (list, dict, tuple)):
            _save_container(child, store, sub, visited, set())


def _save_container(container, store, path, visited, seen_containers):
    if id(container) in seen_containers:
        return
    seen_containers.add(id(container))
    used = {}
    if isinstance(container, dict):
        container = list(container.values())
    for item in container:
        if isinstance(item, Layer):
            # not addressed by `item.name`: names are generated and differ between two
            # instances of one model
            name = _unique_name(to_snake_case(type(item).__name__), used)
            _save_state(item, store, f"{path}/{name}", visited)
        elif isinstance(item, (list, dict, tuple)):
            name = _unique_name("container", used)
            _save_container(item, store, f"{path}/{name}", visited, seen_containers)


class _LoadState:
    def __init__(self, store):
        self.store = store
        self.visited = set()
        self.failed = {}  # id -> (saveable, exception): loaded through no path so far


def _load_state(saveable, st, path="", failed=None):
    """`_load_state` (saving_lib.py:833-945): an object that fails to load under one path
    stays unvisited, so a later path to the same object (a model's `layers` list after a
    nested container) can still load it."""
    failed = st.failed if failed is None else failed
    if id(saveable) in st.visited:
        return
    failure = False
    if hasattr(saveable, "load_own_variables"):
        try:
            saveable.load_own_variables(st.store.get(path))
        except Exception as e:  # recorded, raised at the end if nothing else loads the object
            failed[id(saveable)] = (saveable, e)
            failure = True
    before = len(failed)
    for attr, child in _walk(saveable):
        sub = f"{path}/{attr}" if path else attr
        if isinstance(child, Layer):
            _load_state(child, st, sub, failed)
        elif isinstance(child, (list, dict, tuple)):
            _load_container(child, st, sub, failed, set())
    if not failure:
        if len(failed) - before <= 0:
            st.visited.add(id(saveable))
        failed.pop(id(saveable), None)


def _load_container(container, st, path, failed, seen_containers):
    import warnings

    if id(container) in seen_containers:
        return
    seen_containers.add(id(container))
    used = {}
    if isinstance(container, dict):
        container = list(container.values())
    for item in container:
        if isinstance(item, Layer):
            name = _unique_name(to_snake_case(type(item).__name__), used)
            _load_state(item, st, f"{path}/{name}", failed)
        elif isinstance(item, (list, dict, tuple)):
            name = _unique_name("container", used)
            nested = f"{path}/{name}"
            if not st.store.has_path(nested):
                # files written before nested containers were walked have no such group: try,
                # and warn only if the container held layers that nothing has loaded yet
                tracked = {}
                _load_container(item, st, nested, tracked, seen_containers)
                if tracked:
                    warnings.warn(
                        f"Skipping nested container at '{nested}': no matching group found in "
                        "the saved file. This usually means the file was saved with a Keras "
                        "version that did not serialize sublayers nested inside containers. "
                        "Affected layers will retain their freshly-initialized weights.",
                        stacklevel=2,
                    )
                continue
            _load_container(item, st, nested, failed, seen_containers)


def _load_all(model, store, skip_mismatch=False):
    import warnings

    st = _LoadState(store)
    _load_state(model, st)
    if st.failed:
        first, err = next(iter(st.failed.values()))
        msg = (
            f"A total of {len(st.failed)} objects could not be loaded. Example error message "
            f"for object {first}:\n\n{err}\n\nList of objects that could not be loaded:\n"
            f"{[x[0] for x in st.failed.values()]}"
        )
        if skip_mismatch:
            warnings.warn(msg)
        else:
            raise ValueError(msg)


# ------------------------------------------------------------------------------ weights files


def save_weights(model, filepath, overwrite=True):
    """`model.save_weights("x.weights.h5")` (saving_lib.py:578-633)."""
    import os

    filepath = str(filepath)
    if not filepath.endswith(".weights.h5"):
        raise ValueError(
            "The filename must end in `.weights.h5`. "
            f"Received: filepath={filepath}"
        )
    if os.path.exists(filepath) and not overwrite:
        raise FileExistsError(f"{filepath} exists and `overwrite` is False")
    store = H5Store(filepath, mode="w")
    _save_state(model, store)
    store.close()


def load_weights(model, filepath, skip_mismatch=False):
    """Weights from a `*.weights.h5` file or from the weights member of a `.keras` archive
    (saving_lib.py:636-700)."""
    filepath = str(filepath)
    if filepath.endswith(".weights.h5"):
        store = H5Store(filepath, mode="r")
    elif filepath.endswith(".keras"):
        with zipfile.ZipFile(filepath, "r") as zf:
            store = H5Store(_VARS_FNAME_H5, archive=zf, mode="r")
    else:
        raise ValueError(
            "File format not supported: the filename must end in `.weights.h5` or `.keras`. "
            f"Received: filepath={filepath}"
        )
    _load_all(model, store, skip_mismatch)


# ------------------------------------------------------------------------------ .keras archives

_MODULE_OF = {"Dense": "keras.layers", "EinsumDense": "keras.layers", "Embedding": "keras.layers",
              "ReversibleEmbedding": "keras.layers"}


def serialize_object(obj):
    """The dict `serialize_keras_object` writes for a layer or model
    (keras/src/saving/serialization_lib.py:117-270), for the classes this package has."""
    cls = type(obj)
    module = _MODULE_OF.get(cls.__name__)
    out = {
        "module": module,
        "class_name": cls.__name__,
        "config": obj.get_config(),
        "registered_name": None if module else getattr(cls, "_registered_name", cls.__name__),
    }
    shape = getattr(obj, "_build_input_shape", None)
    if shape is not None:
        out["build_config"] = {"input_shape": list(shape)}
    return out


def _known_classes():
    from keras_amd.layers.dense import Dense
    from keras_amd.layers.einsum_dense import EinsumDense
    from keras_amd.layers.embedding import Embedding, ReversibleEmbedding

    return {c.__name__: c for c in (Dense, EinsumDense, Embedding, ReversibleEmbedding)}


def deserialize_object(config, custom_objects=None, device=None):
    known = _known_classes()
    name = config["class_name"]
    reg = config.get("registered_name")
    custom = custom_objects or {}
    cls = custom.get(reg) or custom.get(name) or (known.get(name) if config.get("module") else None)
    if cls is None:
        raise TypeError(
            f"Could not locate class '{name}'. Make sure custom classes are passed via "
            f"`custom_objects`. Full object config: {config}"
        )
    cfg = dict(config["config"])
    if device is not None:
        cfg["device"] = device
    obj = cls.from_config(cfg) if hasattr(cls, "from_config") else cls(**cfg)
    shape = (config.get("build_config") or {}).get("input_shape")
    if not obj.built and (shape is not None or name in ("Embedding", "ReversibleEmbedding")):
        obj.build(tuple(shape) if shape is not None else None)
    return obj


def save_model(model, filepath, overwrite=True):
    """`model.save("m.keras")`: zip of config.json, metadata.json, model.weights.h5."""
    import os

    filepath = str(filepath)
    if not filepath.endswith(".keras"):
        raise ValueError(
            "Invalid filepath extension for saving. Please add either a `.keras` extension "
            f"for the native Keras format. Received: filepath={filepath}"
        )
    if os.path.exists(filepath) and not overwrite:
        raise FileExistsError(f"{filepath} exists and `overwrite` is False")
    metadata = {"keras_version": KERAS_VERSION,
                "date_saved": datetime.datetime.now().strftime("%Y-%m-%d@%H:%M:%S")}
    with zipfile.ZipFile(filepath, "w") as zf:
        zf.writestr(_METADATA_FILENAME, json.dumps(metadata))
        zf.writestr(_CONFIG_FILENAME, json.dumps(serialize_object(model)))
        store = H5Store(_VARS_FNAME_H5, archive=zf, mode="w")
        _save_state(model, store)
        store.close()


def load_model(filepath, custom_objects=None, device=None):
    """`keras.saving.load_model("m.keras")` for the classes of this package and any classes
    given in `custom_objects` (by registered or class name)."""
    filepath = str(filepath)
    if not filepath.endswith(".keras"):
        raise ValueError(f"File format not supported: filepath={filepath}. Expected a `.keras` file.")
    with zipfile.ZipFile(filepath, "r") as zf:
        config = json.loads(zf.read(_CONFIG_FILENAME))
        model = deserialize_object(config, custom_objects, device)
        store = H5Store(_VARS_FNAME_H5, archive=zf, mode="r")
    _load_all(model, store)
    return model
