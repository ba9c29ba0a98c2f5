"""Several layers on one input.

A decode step calls the query, key and value projections of a block -- and the gate and up
projections of its MLP -- on the same activations.  Each call is a few microseconds of launch
and drain around a kernel that streams a few megabytes, so running them as one launch is worth
more than any tuning of the kernel itself.  The reference has no such call (its layers each run
their own `matmul`); this one returns exactly what the separate calls return.
"""

import contextlib
import threading

import numpy as np
import torch

from keras_amd import ops as kops
from keras_amd.layers.layer import to_torch_dtype

_state = threading.local()

# rows up to which a weight-only int4 layer runs the decode kernel proper (above, other routes)
ADDEND_MAX_ROWS = 16


@contextlib.contextmanager
def shared_input_rows():
    """While active, layers whose activation quantizers are configured alike and that are
    called on the same rows quantise them once (the quantizer is a function of the rows
    alone: keras/src/quantizers/quantizers.py:307-373)."""
    prev = getattr(_state, "memo", None)
    _state.memo = {}
    try:
        yield
    finally:
        _state.memo = prev


def quantize_rows(quantizer, x2):
    """`quantizer(x2, axis=-1)`, taken from the enclosing `shared_input_rows()` when another
    layer has already quantised these very rows with the same settings."""
    memo = getattr(_state, "memo", None)
    config = getattr(quantizer, "get_config", None)
    if memo is None or config is None:
        return quantizer(x2, axis=-1)
    key = _quantizer_key(quantizer, x2)
    hit = memo.get(key)
    if hit is None:
        # the memo keeps x2 alive, so its address cannot be handed to another tensor meanwhile
        hit = memo[key] = (quantizer(x2, axis=-1), x2)
    return hit[0]


def _quantizer_key(quantizer, x2):
    return (type(quantizer), repr(sorted(quantizer.get_config().items())), x2.data_ptr(), tuple(x2.shape),
            tuple(x2.stride()), x2.dtype, x2._version)


def apply_input_op_for(layers, input_op, x):
    """`op(x)` for layers about to be called on it.  Where all of them are int8 layers that quantise
    their input with the same plain abs-max quantizer, the operation and that quantizer run as ONE
    launch and the quantised rows are left in the enclosing `shared_input_rows()` for the layers to
    pick up (same bits as the two launches); otherwise the operation's own launch."""
    from keras_amd import quantizers

    memo = getattr(_state, "memo", None)
    if memo is not None and isinstance(x, torch.Tensor) and x.dim() >= 2:
        qs = [getattr(l, "inputs_quantizer", None) for l in layers]
        first = qs[0] if qs else None
        x2 = x.reshape(-1, x.shape[-1])
        if (first is not None and all(l.quantization_mode == "int8" and type(q) is quantizers.AbsMaxQuantizer
                                      and q.output_dtype == "int8" and q.axis in (None, (-1,))
                                      and q.get_config() == first.get_config() for l, q in zip(layers, qs))
                and kops.input_op_quantize_supported(input_op, x2)):
            h2, q, s = kops.input_op_quantize(input_op, x2, epsilon=first.epsilon, value_range=first.value_range)
            memo[_quantizer_key(first, h2)] = ((q, s), h2)
            return h2.reshape(x.shape)
    return kops.apply_input_op(input_op, x)


def call_together(layers, inputs, input_op=None):
    """`[layer(op(inputs)) for layer in layers]`.

    input_op: None, `("rms_norm", gain, epsilon)` or `("silu_gate", gate)` -- an elementwise /
    row-wise operation between two layers of a decoder block (`ops.rmsnorm`, `ops.silu_mul`).  At
    decode sizes the shared launch applies it to the rows on their way into the kernel, with the
    bits of the separate launch; otherwise it runs as that launch first.

    Weight-only int4 `Dense` / `EinsumDense` layers with one compute dtype, input width and
    group size go to `ops.int4_matmul_multi` (one launch at decode sizes); anything else is
    called layer by layer, with the input rows quantised once for the layers that quantise
    them alike (int8 layers: one quantizer launch instead of one per layer).
    """
    with shared_input_rows():
        return _call_together(layers, inputs, input_op)


def _call_together(layers, inputs, input_op=None):
    layers = list(layers)
    if len(layers) < 2 and input_op is None:
        return [layer(inputs) for layer in layers]
    if not layers:
        return []
    if not isinstance(inputs, torch.Tensor):
        inputs = torch.as_tensor(np.asarray(inputs))
    first = layers[0]
    for layer in layers:
        if not layer.built:
            layer.build(tuple(inputs.shape))
    if any(l.device != first.device or l.compute_dtype != first.compute_dtype for l in layers):
        inputs = apply_input_op_for(layers, input_op, inputs)
        return [layer(inputs) for layer in layers]
    x = inputs.to(first.device) if inputs.device != first.device else inputs
    cd = to_torch_dtype(first.compute_dtype)
    if x.dtype.is_floating_point and x.dtype != cd:
        x = x.to(cd)
    x = x.contiguous()
    # (from here on the layers are handed x: moved and cast once, and the same tensor for all,
    # which is what lets them share its quantised rows)
    # int8 layers at decode sizes that quantise their input alike: one launch from their strip copies
    specs8 = []
    for layer in layers:
        make = getattr(layer, "_int8_together_spec", None)
        spec = make(x) if make is not None else None
        if spec is None:
            break
        specs8.append(spec)
    if (len(specs8) == len(layers)
            and all(s["x2"].shape == specs8[0]["x2"].shape and s["x2"].data_ptr() == specs8[0]["x2"].data_ptr()
                    and s["x2"].stride() == specs8[0]["x2"].stride() and s["settings"] == specs8[0]["settings"]
                    for s in specs8)):
        eps, rng = specs8[0]["settings"]
        quantizer = specs8[0]["quantizer"]
        x2 = specs8[0]["x2"]
        if input_op is not None and all(kops.int8_strip_input_op_supported(
                input_op, x2.shape[0], x2.shape[1], s["kernel"]["units"], rng) for s in specs8):
            outs = kops.int8_dense_strip_multi(x2, [s["kernel"] for s in specs8], epsilon=eps, value_range=rng,
                                               input_op=input_op)
            return [s["finish"](y) for s, y in zip(specs8, outs)]
        if input_op is not None:
            # (the op as a launch of its own; the layers then see a new tensor of the same shape)
            return _call_together(layers, apply_input_op_for(layers, input_op, x))
        outs = kops.int8_dense_strip_multi(x2, [s["kernel"] for s in specs8], epsilon=eps,
                                           value_range=rng, quantize=lambda rows: quantize_rows(quantizer, rows))
        return [s["finish"](y) for s, y in zip(specs8, outs)]
    specs = []
    for layer in layers:
        make = getattr(layer, "_int4_together_spec", None)
        spec = make(x) if make is not None else None
        if spec is None:
            x = apply_input_op_for(layers, input_op, x)
            return [layer(x) for layer in layers]
        specs.append(spec)
    x2 = specs[0]["x2"]
    if x2.shape[0] > 16:
        # beyond decode sizes nothing is shared: every layer takes its own route for the size
        x = apply_input_op_for(layers, input_op, x)
        return [layer(x) for layer in layers]
    if any(s["x2"].shape != x2.shape or s["block_size"] != specs[0]["block_size"] for s in specs):
        x = apply_input_op_for(layers, input_op, x)
        return [layer(x) for layer in layers]
    if input_op is not None and not (
            all(s.get("strip") is not None for s in specs)
            and all(kops.int4_strip_input_op_supported(input_op, x2.shape[0], x2.shape[1], s["strip"]["units"],
                                                       specs[0]["block_size"]) for s in specs)):
        return _call_together(layers, apply_input_op_for(layers, input_op, x))
    if all(s.get("strip") is not None for s in specs):
        # every kernel has its strip-linear copy for these rows: one launch, no scratch
        outs = kops.int4_matmul_strip_multi(x2, [s["strip"] for s in specs], block_size=specs[0]["block_size"],
                                            input_op=input_op)
    else:
        outs = kops.int4_matmul_multi(x2, [s["kernel"] for s in specs], block_size=specs[0]["block_size"])
    return [s["finish"](y) for s, y in zip(specs, outs)]


def _int8_addend_ok(layer, rows, residual):
    """Activation-quantized int8 layer at the rows and widths its decode kernel takes."""
    if layer.quantization_mode != "int8" or not layer.inputs_quantizer or rows > kops.SKINNY_MAX_ROWS:
        return False
    if residual.numel() % rows:
        return False
    units = residual.numel() // rows
    kernel = layer._kernel
    return units % 16 == 0 and (kernel.value.numel() // units) % 8 == 0


def _call_add_with_op(layer, inputs, residual, input_op):
    """`residual + layer(op(inputs))` in one launch where the layer's decode kernel takes the operation
    and a row of addends per row; None where it does not."""
    ok = getattr(layer, "_row_bias_ok", None)
    if not (isinstance(inputs, torch.Tensor) and isinstance(residual, torch.Tensor) and ok is not None
            and layer.built and layer.quantization_mode in ("int8", "int4") and not layer.lora_enabled
            and inputs.is_cuda and inputs.numel() > 0 and residual.device == layer.device
            and inputs.device == layer.device and inputs.dtype == torch.bfloat16
            and residual.dtype == torch.bfloat16 and to_torch_dtype(layer.compute_dtype) == torch.bfloat16 and ok()):
        return None
    x = inputs.contiguous()
    lent = residual.reshape(-1)
    lent = lent if lent.is_contiguous() else lent.contiguous()
    if layer.quantization_mode == "int4":
        make = getattr(layer, "_int4_together_spec", None)
        spec = make(x) if make is not None else None
        if spec is None or spec.get("strip") is None:
            return None
        x2, kernel = spec["x2"], dict(spec["strip"])
        if kernel.get("bias") is not None or lent.numel() != x2.shape[0] * kernel["units"]:
            return None
        if not kops.int4_strip_input_op_supported(input_op, x2.shape[0], x2.shape[1], kernel["units"],
                                                  spec["block_size"]):
            return None
        kernel["bias"] = lent
        (y,) = kops.int4_matmul_strip_multi(x2, [kernel], block_size=spec["block_size"], input_op=input_op,
                                            bias_rows=True)
    else:
        make = getattr(layer, "_int8_together_spec", None)
        spec = make(x) if make is not None else None
        if spec is None:
            return None
        x2, kernel = spec["x2"], dict(spec["kernel"])
        eps, rng = spec["settings"]
        if kernel.get("bias") is not None or lent.numel() != x2.shape[0] * kernel["units"]:
            return None
        if not kops.int8_strip_input_op_supported(input_op, x2.shape[0], x2.shape[1], kernel["units"], rng):
            return None
        kernel["bias"] = lent
        (y,) = kops.int8_dense_strip_multi(x2, [kernel], epsilon=eps, value_range=rng, input_op=input_op,
                                           bias_rows=True)
    out = spec["finish"](y)
    if out.numel() != residual.numel():
        raise ValueError(f"residual of {tuple(residual.shape)} does not match the layer's output {tuple(out.shape)}")
    return out.reshape(residual.shape)


def call_add(layer, inputs, residual, input_op=None):
    """`residual + layer(op(inputs))` (input_op as in `call_together`; None: the inputs as they are).

    For a quantized `Dense` / `EinsumDense` that has neither bias nor activation the add rides
    in the matmul's bias slot: the kernels add a bias to the rounded product,
    `T(T(x . W) + b)`, which is what the separate add computes with `b` = the residual -- the
    same bits, one launch less.  One row: any quantized layer (the residual IS a bias row).
    Up to 16 rows: weight-only int4 layers, up to 8 rows: int8 layers with an activation
    quantizer; their decode kernels take a row of addends per row of x.  Anything else is the
    plain sum.
    """
    if input_op is not None:
        out = _call_add_with_op(layer, inputs, residual, input_op)
        if out is not None:
            return out
        with shared_input_rows():
            return call_add(layer, apply_input_op_for([layer], input_op, inputs), residual)
    ok = getattr(layer, "_row_bias_ok", None)
    if (isinstance(inputs, torch.Tensor) and isinstance(residual, torch.Tensor) and ok is not None
            and layer.built and layer.quantization_mode in ("int8", "int4") and not layer.lora_enabled
            and inputs.numel() > 0 and residual.device == layer.device and inputs.device == layer.device
            and residual.dtype == to_torch_dtype(layer.compute_dtype) and ok()):
        rows = layer._rows_of(inputs)
        if (rows == 1 or (rows <= ADDEND_MAX_ROWS and residual.numel() % rows == 0
                          and layer._int4_together_spec(inputs) is not None)
                or _int8_addend_ok(layer, rows, residual)):
            lent = residual.reshape(-1)
            layer._row_bias = lent if lent.is_contiguous() else lent.contiguous()
            try:
                out = layer(inputs)
            finally:
                layer._row_bias = None
            if out.numel() != lent.numel():
                raise ValueError(f"residual of {tuple(residual.shape)} does not match the layer's "
                                 f"output {tuple(out.shape)}")
            return out.reshape(residual.shape)
    return residual + layer(inputs)
