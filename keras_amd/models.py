"""`Model.quantize`: the caller that converts every layer of a model.

Restates the walk of keras/src/models/model.py:454-699 for the modes built here: visit
the flattened layers, skip nested models, apply `filters`
(keras/src/quantizers/utils.py:4-23), skip layers that are already quantized, treat
`NotImplementedError` from `layer.quantize` as "this layer has no quantized form" and
let every other exception propagate, and return a `QuantizationReport`
(keras/src/quantizers/report.py:12-160).
"""

import re
import warnings
from collections.abc import Callable

from keras_amd.layers.layer import Layer
from keras_amd.quantization_config import validate_and_resolve_config


class QuantizationReport:
    SKIP_NO_SUPPORT = "no quantize support"
    SKIP_FILTERED = "filtered out"
    SKIP_ALREADY_QUANTIZED = "already quantized"
    SKIP_OUTSIDE_STRUCTURE = "outside quantization structure"

    def __init__(self, mode=None):
        self.mode = mode
        self.quantized = []  # (path, mode, dtype-policy name)
        self.skipped = []    # (path, reason)
        self.errors = []     # (path, message)

    def add_quantized(self, path, mode, scheme):
        self.quantized.append((path, mode, scheme))

    def add_skipped(self, path, reason):
        self.skipped.append((path, reason))

    def add_error(self, path, error):
        self.errors.append((path, str(error)))

    @property
    def num_quantized(self):
        return len(self.quantized)

    @property
    def num_skipped(self):
        return len(self.skipped)

    @property
    def num_errors(self):
        return len(self.errors)

    def skipped_by_reason(self, reason):
        return [path for path, r in self.skipped if r == reason]

    def summary_warning(self, max_examples=5):
        unsupported = self.skipped_by_reason(self.SKIP_NO_SUPPORT)
        if not unsupported and not self.errors:
            return None
        parts = []
        if unsupported:
            examples = ", ".join(repr(p) for p in unsupported[:max_examples])
            if len(unsupported) > max_examples:
                examples += ", ..."
            parts.append(
                f"{len(unsupported)} layer(s) were skipped because they do "
                f"not support quantization (e.g. {examples})."
            )
        if self.errors:
            examples = ", ".join(repr(p) for p, _ in self.errors[:max_examples])
            if len(self.errors) > max_examples:
                examples += ", ..."
            parts.append(f"{len(self.errors)} layer(s) reported errors (e.g. {examples}).")
        parts.append(
            f"Quantized {self.num_quantized} layer(s) in mode "
            f"'{self.mode}'. Call `model.quantization_summary()` or inspect "
            "the returned `QuantizationReport` for details."
        )
        return "`model.quantize()`: " + " ".join(parts)

    def render(self):
        lines = [f"Quantization report (mode='{self.mode}')"]
        lines.append(f"  quantized: {self.num_quantized}")
        for path, mode, scheme in self.quantized:
            lines.append(f"    {path}: {mode} ({scheme})")
        lines.append(f"  skipped: {self.num_skipped}")
        for path, reason in self.skipped:
            lines.append(f"    {path}: {reason}")
        if self.errors:
            lines.append(f"  errors: {self.num_errors}")
            for path, message in self.errors:
                lines.append(f"    {path}: {message}")
        return "\n".join(lines)


def should_quantize_layer(layer, filters):
    """keras/src/quantizers/utils.py:4-23."""
    if filters is None:
        return True
    if isinstance(filters, str):
        return bool(re.search(filters, layer.name))
    if isinstance(filters, (list, tuple)):
        return any(re.search(pat, layer.name) for pat in filters)
    if callable(filters):
        return filters(layer)
    return True


def _sublayers(obj, seen):
    """Layers held in attributes (directly or inside lists / tuples / dicts), depth first,
    in attribute order -- what `Layer._flatten_layers(include_self=False)` yields."""
    out = []

    def visit(value):
        if isinstance(value, Layer):
            if id(value) in seen:
                return
            seen.add(id(value))
            out.append(value)
            out.extend(_sublayers(value, seen))
        elif isinstance(value, (list, tuple)):
            for v in value:
                visit(v)
        elif isinstance(value, dict):
            for v in value.values():
                visit(v)

    for key, value in vars(obj).items():
        if key.startswith("__"):
            continue
        visit(value)
    return out


class Model(Layer):
    """A layer that owns layers; only the part of `keras.Model` that `quantize` needs."""

    def __init__(self, dtype=None, name=None, device=None):
        super().__init__(dtype=dtype, name=name, device=device)
        self.built = True
        self._quantization_report = None

    def _flatten_layers(self, include_self=False):
        seen = {id(self)}
        layers = _sublayers(self, seen)
        return ([self] if include_self else []) + layers

    def resident_bytes(self):
        """`Layer.resident_bytes` summed over the model and every layer below it."""
        total = {"stored": 0, "derived": 0}
        for layer in self._flatten_layers(include_self=True):
            part = Layer.resident_bytes(layer)
            total["stored"] += part["stored"]
            total["derived"] += part["derived"]
        return total

    @property
    def layers(self):
        """The layers held directly by this model, containers flattened, sublayers of layers
        not descended into (keras/src/models/model.py:174-176:
        `_flatten_layers(include_self=False, recursive=False)`)."""
        out, seen = [], {id(self)}

        def visit(value):
            if isinstance(value, Layer):
                if id(value) not in seen:
                    seen.add(id(value))
                    out.append(value)
            elif isinstance(value, (list, tuple)):
                for v in value:
                    visit(v)
            elif isinstance(value, dict):
                for v in value.values():
                    visit(v)

        for key, value in vars(self).items():
            if not key.startswith("__"):
                visit(value)
        return out

    # ---- saving (keras/src/models/model.py:save / save_weights / load_weights) ----------
    def save(self, filepath, overwrite=True):
        from keras_amd import saving

        saving.save_model(self, filepath, overwrite=overwrite)

    def save_weights(self, filepath, overwrite=True):
        from keras_amd import saving

        saving.save_weights(self, filepath, overwrite=overwrite)

    def load_weights(self, filepath):
        from keras_amd import saving

        saving.load_weights(self, filepath)

    def get_config(self):
        return {"name": self.name, "dtype": self.dtype_policy.name}

    def quantize(self, mode=None, config=None, filters=None, verbose=False, **kwargs):
        type_check = kwargs.pop("type_check", True)
        if kwargs:
            raise ValueError(
                f"Unrecognized keyword arguments passed to {self.__class__.__name__}: {kwargs}"
            )
        if filters is not None and not isinstance(filters, (str, Callable, list, tuple)):
            raise ValueError(
                "The `filters` argument must be a regex string, a list of "
                f"regex strings, or a callable. Received: {type(filters)}"
            )
        config = validate_and_resolve_config(mode, config)
        mode = config.mode
        report = QuantizationReport(mode=mode)
        for layer in self._flatten_layers():
            if isinstance(layer, Model):
                continue  # its layers are visited by this walk already
            path = getattr(layer, "path", None) or layer.name
            if not should_quantize_layer(layer, filters):
                report.add_skipped(path, QuantizationReport.SKIP_FILTERED)
                continue
            if getattr(layer, "_is_quantized", False):
                report.add_skipped(path, QuantizationReport.SKIP_ALREADY_QUANTIZED)
                continue
            try:
                layer.quantize(mode, type_check=type_check, config=config)
            except NotImplementedError:
                report.add_skipped(path, QuantizationReport.SKIP_NO_SUPPORT)
                continue
            report.add_quantized(path, layer.quantization_mode, layer.dtype_policy.name)
        message = report.summary_warning()
        if message is not None:
            warnings.warn(message, stacklevel=2)
        if verbose:
            print(report.render())
        self._quantization_report = report
        return report
