"""GPU: Model.quantize over a small Llama-style decoder, and the decoder's quantized forward
against a CPU forward that calls the oracle for every weight-carrying layer."""

import warnings

import pytest
import torch

from keras_amd.decoder_harness import LlamaStyleDecoder, apply_rope, rope_tables
from keras_amd.models import QuantizationReport
from oracle import keras_cpu_path as ref
from tests.helpers import max_rel_err

pytestmark = pytest.mark.gpu

CFG = dict(vocab=500, d_model=128, n_heads=4, ffn_dim=256, n_layers=2, max_len=32)


def cpu(var):
    return var.value.cpu()


def oracle_layer(layer, x):
    """One Dense / EinsumDense call on the CPU through the oracle, from the layer's variables."""
    mode = layer.quantization_mode
    eq = getattr(layer, "equation", None)
    cd = layer.compute_dtype
    if mode is None:
        k = cpu(layer._kernel)
        return torch.einsum(eq, x, k) if eq else x @ k
    if mode == "int8":
        if eq:
            return ref.einsum_dense_int8_call(x, cpu(layer._kernel), cpu(layer.kernel_scale), eq,
                                              compute_dtype=cd)
        return ref.dense_int8_call(x, cpu(layer._kernel), cpu(layer.kernel_scale), compute_dtype=cd)
    bs = layer._int4_block_size
    grouped = bs is not None and bs > 0
    zero = cpu(layer.kernel_zero) if grouped else None
    g_idx = cpu(layer.g_idx) if grouped else None
    if eq:
        qk = dict(kernel=cpu(layer._kernel), kernel_scale=cpu(layer.kernel_scale), kernel_zero=zero,
                  g_idx=g_idx, cols=layer._int4_unpacked_column_size,
                  original_kernel_shape=layer.original_kernel_shape)
        return ref.einsum_dense_int4_call(x, qk, eq, compute_dtype=cd, block_size=bs)
    return ref.dense_int4_call(x, cpu(layer._kernel), cpu(layer.kernel_scale), layer._orig_output_dim,
                               kernel_zero=zero, g_idx=g_idx, block_size=bs, compute_dtype=cd)


def oracle_forward(model, ids):
    """Full-sequence causal forward on the CPU: logits [B, T, vocab]."""
    emb = model.token_embedding
    B, T = ids.shape
    if emb.quantization_mode == "int8":
        x = ref.embedding_int8_call(ids, cpu(emb._embeddings), cpu(emb.embeddings_scale),
                                    compute_dtype=emb.compute_dtype)
    elif emb.quantization_mode is None:
        x = cpu(emb._embeddings)[ids]
    else:
        bs = emb._int4_block_size
        grouped = bs is not None and bs > 0
        x = ref.embedding_int4_call(
            ids, cpu(emb._embeddings), cpu(emb.embeddings_scale), emb.output_dim,
            embeddings_zero=cpu(emb.embeddings_zero) if grouped else None,
            g_idx=cpu(emb.g_idx) if grouped else None, block_size=bs,
            compute_dtype=emb.compute_dtype)
    cos, sin = rope_tables(model.head_dim, model.max_len, torch.device("cpu"), dtype=x.dtype)
    cos, sin = cos[:T], sin[:T]
    causal = torch.ones(T, T, dtype=torch.bool).tril()

    def norm(layer, v):
        return torch.nn.functional.rms_norm(v, (layer.dim,), cpu(layer.scale).to(v.dtype), layer.epsilon)

    for blk in model.blocks:
        h = norm(blk.attn_norm, x)
        q = apply_rope(oracle_layer(blk.query, h), cos, sin)
        k = apply_rope(oracle_layer(blk.key, h), cos, sin)
        v = oracle_layer(blk.value, h)
        a = torch.nn.functional.scaled_dot_product_attention(
            q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask=causal[None, None])
        x = x + oracle_layer(blk.attn_out, a.transpose(1, 2))
        h = norm(blk.ffn_norm, x)
        x = x + oracle_layer(blk.down, torch.nn.functional.silu(oracle_layer(blk.gate, h))
                             * oracle_layer(blk.up, h))
    x = norm(model.final_norm, x)
    if emb.quantization_mode == "int8":
        return ref.reversible_embedding_int8_reverse(
            x.reshape(B * T, -1), cpu(emb._embeddings), cpu(emb.embeddings_scale),
            compute_dtype=emb.compute_dtype).reshape(B, T, -1)
    if emb.quantization_mode == "int4":
        bs = emb._int4_block_size
        grouped = bs is not None and bs > 0
        return ref.reversible_embedding_int4_reverse(
            x.reshape(B * T, -1), cpu(emb._embeddings), cpu(emb.embeddings_scale), emb.output_dim,
            embeddings_zero=cpu(emb.embeddings_zero) if grouped else None,
            g_idx=cpu(emb.g_idx) if grouped else None, block_size=bs,
            compute_dtype=emb.compute_dtype).reshape(B, T, -1)
    return x @ cpu(emb._embeddings).T


def quantize(model, mode):
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        return model.quantize(mode)


@pytest.mark.parametrize("mode", ["int8", "int4"])
def test_model_quantize_report(dev, mode):
    model = LlamaStyleDecoder(dtype="float32", device=dev, **CFG)
    report = quantize(model, mode)
    per_block = 7
    n_q = per_block * CFG["n_layers"] + 1
    assert report.mode == mode and report.num_quantized == n_q
    # norms (2 per block + final) and the blocks themselves have no quantized form
    unsupported = report.skipped_by_reason(QuantizationReport.SKIP_NO_SUPPORT)
    assert len(unsupported) == 3 * CFG["n_layers"] + 1
    if mode == "int4":
        assert all(s == "int4/128_from_float32" for _, _, s in report.quantized)
    model2 = LlamaStyleDecoder(dtype="float32", device=dev, **CFG)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        filtered = model2.quantize(mode, filters=lambda l: l.name != "token_embedding")
    assert filtered.skipped_by_reason(QuantizationReport.SKIP_FILTERED) == ["token_embedding"]
    assert filtered.num_quantized == n_q - 1
    again = quantize(model, mode)
    assert again.num_quantized == 0
    assert len(again.skipped_by_reason(QuantizationReport.SKIP_ALREADY_QUANTIZED)) == n_q
    with pytest.raises(ValueError):
        model.quantize(mode, filters=3)
    with pytest.raises(ValueError):
        model.quantize(mode, bogus=1)


@pytest.mark.parametrize("mode", [None, "int8", "int4"])
def test_decoder_forward_matches_cpu(dev, mode):
    model = LlamaStyleDecoder(dtype="float32", device=dev, **CFG)
    if mode:
        quantize(model, mode)
    ids = torch.randint(0, CFG["vocab"], (2, 9), generator=torch.Generator().manual_seed(1))
    cache = model.new_cache(2)
    logits = model.forward(ids.to(dev), torch.arange(9, device=dev), cache, last_only=False)
    want = oracle_forward(model, ids)
    assert tuple(logits.shape) == (2, 9, CFG["vocab"])
    # dynamic activation quantisation can flip a rounding when the float glue differs in the
    # last bit between CPU and GPU; a flipped int8 step is ~1/127 of one activation
    tol = 2e-2 if mode == "int8" else 1e-3
    assert max_rel_err(logits, want) <= tol
    # one more position through the cache == the same position of a full-sequence forward
    nxt = torch.randint(0, CFG["vocab"], (2, 1), generator=torch.Generator().manual_seed(2))
    step = model.forward(nxt.to(dev), torch.tensor([9], device=dev), cache)
    full = oracle_forward(model, torch.cat([ids, nxt], dim=1))[:, -1:, :]
    assert max_rel_err(step, full) <= tol


@pytest.mark.parametrize("mode,dtype", [("int8", "float32"), ("int4", "bfloat16"), ("int8", "bfloat16")])
def test_generate_graph_equals_eager(dev, mode, dtype):
    model = LlamaStyleDecoder(dtype=dtype, device=dev, **CFG)
    quantize(model, mode)
    prompt = torch.randint(0, CFG["vocab"], (3, 8), generator=torch.Generator().manual_seed(3))
    eager = model.generate(prompt, 12, use_graph=False)
    graphed = model.generate(prompt, 12, use_graph=True)
    assert tuple(eager.shape) == (3, 12)
    assert torch.equal(eager.cpu(), graphed.cpu())
    again = model.generate(prompt, 12, use_graph=True)
    assert torch.equal(graphed.cpu(), again.cpu())
    # the prompt graph and the step graph are kept by the model and only replayed from here on:
    # other prompts of the same shape, another prompt length and fewer steps, with eager work
    # and synchronisations between the replays, each against the eager result
    for seed, shape, steps in [(5, (3, 8), 12), (6, (3, 8), 7), (7, (3, 20), 9), (8, (3, 8), 12),
                               (9, (3, 20), 9), (3, (3, 8), 12)]:
        other = torch.randint(0, CFG["vocab"], shape, generator=torch.Generator().manual_seed(seed))
        want = model.generate(other, steps, use_graph=False)
        torch.cuda.synchronize()
        got = model.generate(other, steps, use_graph=True)
        assert tuple(got.shape) == (3, steps)
        assert torch.equal(want.cpu(), got.cpu()), (seed, shape, steps)
    assert torch.equal(model.generate(prompt, 12, use_graph=True).cpu(), eager.cpu())


def test_generate_graphs_follow_weight_changes(dev):
    model = LlamaStyleDecoder(dtype="bfloat16", device=dev, layer_policy="int4/128_from_bfloat16",
                              **{**CFG, "d_model": 256, "ffn_dim": 512})
    model.randomize_quantized_weights(seed=1)
    prompt = torch.randint(0, CFG["vocab"], (2, 20), generator=torch.Generator().manual_seed(4))
    first = model.generate(prompt, 8, use_graph=True)
    assert torch.equal(first.cpu(), model.generate(prompt, 8, use_graph=False).cpu())
    model.randomize_quantized_weights(seed=2)   # the kept graphs point at the old derived copies
    want = model.generate(prompt, 8, use_graph=False)
    got = model.generate(prompt, 8, use_graph=True)
    assert torch.equal(want.cpu(), got.cpu())
    assert not torch.equal(first.cpu(), got.cpu())


@pytest.mark.parametrize("policy", ["int4/128_from_bfloat16", "int4/-1_from_bfloat16", "int8_from_bfloat16"])
def test_prebuilt_quantized_decoder_runs(dev, policy):
    model = LlamaStyleDecoder(dtype="bfloat16", device=dev, layer_policy=policy,
                              **{**CFG, "d_model": 256, "ffn_dim": 512})
    mode = policy[:4]
    assert model.blocks[0].gate.quantization_mode == mode
    assert model.blocks[0].gate._kernel.dtype == "int8"
    assert model.token_embedding.quantization_mode == mode
    model.randomize_quantized_weights()
    prompt = torch.randint(0, CFG["vocab"], (2, 8), generator=torch.Generator().manual_seed(4))
    stats = {}
    out = model.generate(prompt, 6, stats=stats)
    assert tuple(out.shape) == (2, 6) and int(out.min()) >= 0 and int(out.max()) < CFG["vocab"]
    assert stats["decode_steps"] == 4 and stats["decode_ms"] > 0


FULL_WIDTH = dict(vocab=2048, d_model=4096, n_heads=32, ffn_dim=14336, max_len=64)


@pytest.mark.parametrize("policy", ["int4/128_from_bfloat16", "int8_from_bfloat16"])
def test_full_width_block_matches_cpu(dev, policy):
    # one decoder block at the width of target configuration 5 (d_model 4096, 32 heads, SwiGLU
    # 14336; a small vocabulary keeps the CPU side short), bfloat16, synthetic quantized weights:
    # a 48-row prompt forward (the mid-sized kernels) and one cached step of 2 rows (the decode
    # kernels) against the CPU forward through the oracle
    model = LlamaStyleDecoder(dtype="bfloat16", device=dev, layer_policy=policy, n_layers=1, **FULL_WIDTH)
    model.randomize_quantized_weights(seed=5)
    g = torch.Generator().manual_seed(21)
    ids = torch.randint(0, FULL_WIDTH["vocab"], (2, 24), generator=g)
    cache = model.new_cache(2)
    logits = model.forward(ids.to(dev), torch.arange(24, device=dev), cache, last_only=False)
    want = oracle_forward(model, ids)
    assert tuple(logits.shape) == (2, 24, FULL_WIDTH["vocab"])
    assert torch.isfinite(want).all() and want.abs().max() > 0
    # bfloat16 end to end: every op's result is rounded to 8 bits of significand on both sides,
    # and the float glue (norms, RoPE, softmax) differs in the last bit between CPU and GPU; with
    # int8 layers such a bit also moves activations across quantisation steps, and the moved steps
    # pass through three more quantised layers.  The layers themselves are held to the oracle on
    # identical inputs below, bit for bit where they are integer work.
    tol = 5e-2 if policy.startswith("int8") else 1e-2
    err = max_rel_err(logits, want)
    print(f"full-width block {policy}: prompt err {err:.3e}", flush=True)
    assert err <= tol
    nxt = torch.randint(0, FULL_WIDTH["vocab"], (2, 1), generator=g)
    step = model.forward(nxt.to(dev), torch.tensor([24], device=dev), cache)
    full = oracle_forward(model, torch.cat([ids, nxt], dim=1))[:, -1:, :]
    err = max_rel_err(step, full)
    print(f"full-width block {policy}: cached step err {err:.3e}", flush=True)
    assert err <= tol

    # every weight-carrying layer of the block on the same inputs as the oracle: alone, and through
    # the shared-input / residual entry points the block uses, at 48 rows and at 2 rows
    from keras_amd.layers import call_add, call_together

    blk = model.blocks[0]
    bits = lambda t: t.contiguous().view(torch.int16)

    def check(got, want_cpu, what):
        if policy.startswith("int8"):
            assert torch.equal(bits(got.cpu()), bits(want_cpu)), what
        else:
            assert max_rel_err(got, want_cpu) <= 1e-2, what

    for T in (24, 1):
        h = torch.randn(2, T, 4096, generator=g).to(torch.bfloat16)
        a = torch.randn(2, T, 32, 128, generator=g).to(torch.bfloat16)
        f = torch.randn(2, T, 14336, generator=g).to(torch.bfloat16)
        res = torch.randn(2, T, 4096, generator=g).to(torch.bfloat16)
        h_d, a_d, f_d, res_d = h.to(dev), a.to(dev), f.to(dev), res.to(dev)
        want_h = {n: oracle_layer(getattr(blk, n), h) for n in ("query", "key", "value", "gate", "up")}
        for n, w in want_h.items():
            check(getattr(blk, n)(h_d), w, (T, n))
        for names in (("query", "key", "value"), ("gate", "up")):
            outs = call_together(tuple(getattr(blk, n) for n in names), h_d)
            for n, y in zip(names, outs):
                check(y, want_h[n], (T, "together", n))
        want_o, want_d = oracle_layer(blk.attn_out, a), oracle_layer(blk.down, f)
        check(blk.attn_out(a_d), want_o, (T, "attn_out"))
        check(blk.down(f_d), want_d, (T, "down"))
        check(call_add(blk.attn_out, a_d, res_d), res + want_o, (T, "attn_out+residual"))
        check(call_add(blk.down, f_d, res_d), res + want_d, (T, "down+residual"))


@pytest.mark.parametrize("policy", ["int4/128_from_bfloat16", "int8_from_bfloat16"])
def test_full_size_generate_graph_equals_eager(dev, policy):
    # target configuration 5 at full size: 32 layers, d_model 4096, 32 heads, SwiGLU 14336, vocabulary
    # 32000; the tokens of the HIP-graph replay are the tokens of the eager loop
    model = LlamaStyleDecoder(max_len=64, dtype="bfloat16", device=dev, layer_policy=policy)
    assert (len(model.blocks), model.d_model, model.vocab) == (32, 4096, 32000)
    model.randomize_quantized_weights(seed=9)
    prompt = torch.randint(0, model.vocab, (2, 16), generator=torch.Generator().manual_seed(31))
    eager = model.generate(prompt, 6, use_graph=False)
    graphed = model.generate(prompt, 6, use_graph=True)
    assert tuple(eager.shape) == (2, 6)
    assert torch.equal(eager.cpu(), graphed.cpu())
    torch.cuda.synchronize()
    other = torch.randint(0, model.vocab, (2, 16), generator=torch.Generator().manual_seed(32))
    want = model.generate(other, 6, use_graph=False)
    got = model.generate(other, 6, use_graph=True)
    assert torch.equal(want.cpu(), got.cpu())
    del model
    torch.cuda.empty_cache()
