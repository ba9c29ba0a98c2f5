"""Llama-style decoder assembled from the quantizable layer mirrors: the caller of the path.

Every weight matrix of the network sits in a `Dense`, `EinsumDense` or
`ReversibleEmbedding`, so after `model.quantize("int8" | "int4")` every matmul of a
forward pass goes through the k3q kernels; what is left to torch is glue that the
reference also leaves to backend ops (RMS norm, rotary embedding, softmax attention over
the KV cache, SwiGLU gating, residual adds, argmax).

Shape of the network (d_model, heads, ffn, vocab, layers) follows the usual Llama layout:
pre-norm blocks, attention projections as einsum layers `btd,dnh->btnh` / `btnh,nhd->btd`,
a gated feed-forward of three Dense layers, tied input / output embeddings.
"""

import math

import torch

from keras_amd import dtype_policies, ops as kops
from keras_amd.layers import Dense, EinsumDense, ReversibleEmbedding, call_add, call_together
from keras_amd.layers.layer import Layer, as_tensor, to_torch_dtype
from keras_amd.models import Model
from keras_amd.quantization_config import Int4QuantizationConfig


class RMSNorm(Layer):
    def __init__(self, dim, epsilon=1e-6, dtype=None, name=None, device=None):
        super().__init__(dtype=dtype, name=name, device=device)
        self.dim = dim
        self.epsilon = epsilon
        self.build((None, dim))

    def build(self, input_shape):
        self.scale = self.add_weight(name="scale", shape=(self.dim,), initializer="ones", trainable=True)
        self.built = True

    def as_input_op(self):
        """This layer as the `input_op` of `call_together` / `call_add`."""
        return ("rms_norm", self.read(self.scale), self.epsilon)

    def call(self, x, training=None):
        w = self.read(self.scale)
        if x.numel() <= (64 << 10) and kops.rmsnorm_supported(x, w):
            return kops.rmsnorm(x, w, self.epsilon)  # decode sizes: one short launch
        return torch.nn.functional.rms_norm(x, (self.dim,), w, self.epsilon)


def _silu_mul(gate, up):
    if gate.numel() <= (256 << 10) and kops.silu_mul_supported(gate, up):
        return kops.silu_mul(gate, up)
    return torch.nn.functional.silu(gate) * up


def rope_tables(head_dim, max_len, device, base=10000.0, dtype=torch.float32):
    """cos / sin [max_len, head_dim] for the rotate-half form: the half-width table repeated,
    the first half of sin negated (the sign of the rotated half lives in the table, so
    applying it costs no negation)."""
    inv = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    ang = torch.outer(torch.arange(max_len, dtype=torch.float32), inv)
    cos = torch.cos(torch.cat((ang, ang), dim=-1))
    sin = torch.cat((-torch.sin(ang), torch.sin(ang)), dim=-1)
    return cos.to(device=device, dtype=dtype), sin.to(device=device, dtype=dtype)


def apply_rope(x, cos, sin):
    """x [B, T, H, hd]; cos / sin [T, hd] from `rope_tables` for the positions of these T
    tokens (rotate-half: pairs are (i, i + hd/2); x * cos + (-x2, x1) * |sin|)."""
    half = x.shape[-1] // 2
    swapped = torch.cat((x[..., half:], x[..., :half]), dim=-1)
    return x * cos[None, :, None, :] + swapped * sin[None, :, None, :]


class DecoderBlock(Layer):
    def __init__(self, d_model, n_heads, ffn_dim, dtype=None, layer_dtype=None, name=None,
                 device=None, init=None):
        """dtype: policy of the block and its norms; layer_dtype: policy of the
        weight-carrying layers (a quantized policy name builds them already quantized)."""
        super().__init__(dtype=dtype, name=name, device=device)
        hd = d_model // n_heads
        kw = dict(dtype=layer_dtype or dtype, device=device, kernel_initializer=init)
        self.n_heads, self.head_dim = n_heads, hd
        self.attn_norm = RMSNorm(d_model, dtype=dtype, device=device, name=f"{name}_attn_norm")
        self.query = EinsumDense("btd,dnh->btnh", (None, n_heads, hd), name=f"{name}_query", **kw)
        self.key = EinsumDense("btd,dnh->btnh", (None, n_heads, hd), name=f"{name}_key", **kw)
        self.value = EinsumDense("btd,dnh->btnh", (None, n_heads, hd), name=f"{name}_value", **kw)
        self.attn_out = EinsumDense("btnh,nhd->btd", (None, d_model), name=f"{name}_attn_out", **kw)
        self.ffn_norm = RMSNorm(d_model, dtype=dtype, device=device, name=f"{name}_ffn_norm")
        self.gate = Dense(ffn_dim, use_bias=False, name=f"{name}_ffn_gate", **kw)
        self.up = Dense(ffn_dim, use_bias=False, name=f"{name}_ffn_up", **kw)
        self.down = Dense(d_model, use_bias=False, name=f"{name}_ffn_down", **kw)
        for layer in (self.query, self.key, self.value):
            layer.build((None, None, d_model))
        self.attn_out.build((None, None, n_heads, hd))
        self.gate.build((None, d_model))
        self.up.build((None, d_model))
        self.down.build((None, ffn_dim))
        self.built = True

    def forward(self, x, rows, cache, pos, tables=None, oob_flag=None):
        """x [B, T, D].  cache: (k, v) each [B, H, maxT, hd], written at positions `pos`
        (an int64 device tensor [T]); rows(): (cos, sin, mask) of these positions -- the table
        rows and mask [T, maxT], 0 where a key may be attended to, -inf elsewhere -- asked for
        only by the torch path; tables: the whole (cos, sin) tables, for the one-position kernel;
        oob_flag: the int32 device flag that kernel raises for a position outside the cache."""
        # The normalisations and the gate are handed to the projections that consume them as their
        # `input_op`: at one position they ride inside the projections' launches, in front of int8
        # layers they share a launch with the activation quantizer, otherwise they run as their own
        # kernels (same bits every way).
        fused = x.is_cuda and x.dtype == torch.bfloat16
        if fused:
            q, k, v = call_together((self.query, self.key, self.value), x, input_op=self.attn_norm.as_input_op())
        else:
            q, k, v = call_together((self.query, self.key, self.value), self.attn_norm(x))
        if tables is not None and q.shape[1] == 1 and kops.decode_attention_supported(q, cache[0]):
            # one position: rotation, cache update and attention in one launch (5 launches per block)
            a = kops.decode_attention(q, k, v, tables[0], tables[1], pos, cache[0], cache[1], oob_flag=oob_flag)
        else:
            # one rotation over the query and key heads together (half the elementwise launches)
            cos, sin, mask = rows()
            qk = apply_rope(torch.cat((q, k), dim=2), cos, sin)
            q, k = qk[:, :, : self.n_heads], qk[:, :, self.n_heads:]
            kc, vc = cache
            kc.index_copy_(2, pos, k.transpose(1, 2))
            vc.index_copy_(2, pos, v.transpose(1, 2))
            a = torch.nn.functional.scaled_dot_product_attention(
                q.transpose(1, 2), kc, vc, attn_mask=mask[None, None]).transpose(1, 2)
        # (the residual rides in the projection's bias slot where it can, same bits as the add)
        x = call_add(self.attn_out, a, x)
        if fused:
            gate, up = call_together((self.gate, self.up), x, input_op=self.ffn_norm.as_input_op())
            return call_add(self.down, up, x, input_op=("silu_gate", gate))
        gate, up = call_together((self.gate, self.up), self.ffn_norm(x))
        return call_add(self.down, _silu_mul(gate, up), x)


class LlamaStyleDecoder(Model):
    def __init__(self, vocab=32000, d_model=4096, n_heads=32, ffn_dim=14336, n_layers=32,
                 max_len=256, dtype="bfloat16", device=None, seed=0, layer_policy=None,
                 init_on_device=False):
        """layer_policy: dtype-policy name for the weight-carrying layers, e.g.
        "int4/128_from_bfloat16": the layers are then built already quantized (zero
        weights, to be filled by `load_own_variables` or `randomize_quantized_weights`)
        instead of being built in float and converted.
        init_on_device: draw the random initial weights with the device's generator instead of
        the host's (seconds instead of half a minute at full size; another stream of numbers)."""
        super().__init__(dtype=dtype, name="llama_style_decoder", device=device)
        self.vocab, self.d_model, self.n_heads = vocab, d_model, n_heads
        self.head_dim = d_model // n_heads
        self.max_len = max_len
        gen_device = self.device if init_on_device else torch.device("cpu")
        gen = torch.Generator(device=gen_device).manual_seed(seed)
        wdtype = layer_policy or dtype

        def init(shape, dt):
            # N(0, 1/fan_in); the output projection [heads, head_dim, d_model] contracts its
            # two leading axes, every other kernel its first
            fan_in = shape[0] * shape[1] if len(shape) == 3 and shape[0] == n_heads else shape[0]
            return (torch.randn(shape, generator=gen, device=gen_device) * (1.0 / math.sqrt(fan_in))).to(dt)

        # A layer built straight from an int4 policy has no config and would fall back to the
        # default activation quantizer (reversible_embedding.py:229-233); pass the config that
        # `quantize("int4")` resolves to, so that both construction paths give the same layer.
        emb_config = None
        policy = dtype_policies.get(wdtype)
        if policy.quantization_mode == "int4":
            emb_config = Int4QuantizationConfig(block_size=policy.block_size)
        self.token_embedding = ReversibleEmbedding(
            vocab, d_model, dtype=wdtype, device=self.device, name="token_embedding",
            quantization_config=emb_config,
            embeddings_initializer=lambda s, dt: (torch.randn(s, generator=gen, device=gen_device) * 0.02).to(dt))
        self.token_embedding.build()
        self.token_embedding.check_ids = False
        self.blocks = [
            DecoderBlock(d_model, n_heads, ffn_dim, dtype=dtype, layer_dtype=wdtype,
                         device=self.device, name=f"block{i}", init=init)
            for i in range(n_layers)
        ]
        self.final_norm = RMSNorm(d_model, dtype=dtype, device=self.device, name="final_norm")
        self.cos, self.sin = rope_tables(self.head_dim, max_len, self.device,
                                         dtype=to_torch_dtype(self.compute_dtype))
        self._graphs = {}
        # raised by the one-position attention kernel when a step's position is outside the cache
        # (the torch path's index_copy_ raises there); read by check_positions()
        self._pos_oob = torch.zeros(1, dtype=torch.int32, device=self.device)

    def check_positions(self):
        """Raise IndexError if any decode step since the last check ran at a position outside
        the cache (synchronises)."""
        if int(self._pos_oob.item()):
            self._pos_oob.zero_()
            raise IndexError(f"a decode step ran at a position outside the cache of {self.max_len} rows")

    # ---- synthetic quantized weights ---------------------------------------------------
    def randomize_quantized_weights(self, seed=0):
        """Fill already-quantized layers with random int8 / packed-int4 values and plausible
        scales, on the device (throughput runs at sizes where converting float weights on
        the host would take minutes).  Values are not a quantisation of anything."""
        g = torch.Generator(device=self.device).manual_seed(seed)
        for layer in self._flatten_layers():
            for var in getattr(layer, "_variables", []):
                t = as_tensor(var)
                short = var.name.rsplit("/", 1)[-1]
                if short == "g_idx":
                    continue
                if t.dtype == torch.int8 and short.endswith("zero"):
                    var.assign(torch.randint(-2, 3, t.shape, generator=g, device=self.device, dtype=torch.int8))
                elif t.dtype == torch.int8:
                    var.assign(torch.randint(-128, 128, t.shape, generator=g, device=self.device, dtype=torch.int8))
                elif short.endswith("_scale"):
                    # keep de-quantised magnitudes near 1/sqrt(fan_in) so activations stay finite
                    grouped = (getattr(layer, "_int4_block_size", None) or -1) > 0
                    u = torch.rand(t.shape, generator=g, device=self.device)
                    if layer.quantization_mode == "int4" and grouped:
                        v = u * 0.002 + 0.002       # value = (q - zero) * scale
                    elif layer.quantization_mode == "int4":
                        v = u * 200.0 + 300.0       # value = q / scale, |q| <= 8
                    else:
                        v = u * 2000.0 + 4000.0     # value = q / scale, |q| <= 127
                    var.assign(v.to(t.dtype))

    # ---- forward ---------------------------------------------------------------------------
    def new_cache(self, batch):
        cd = to_torch_dtype(self.compute_dtype)
        shape = (batch, self.n_heads, self.max_len, self.head_dim)
        return [(torch.zeros(shape, dtype=cd, device=self.device),
                 torch.zeros(shape, dtype=cd, device=self.device)) for _ in self.blocks]

    def forward(self, ids, pos, cache, last_only=True):
        """ids [B, T] token ids at positions pos [T] (int64 device tensor) -> logits."""
        x = self.token_embedding(ids)
        cd = to_torch_dtype(self.compute_dtype)
        if x.dtype != cd:
            x = x.to(cd)
        made = []

        def rows():
            # table rows and mask of these positions, made once per forward and only if a block
            # asks (a step on the one-position kernel does not: six small launches less)
            if not made:
                cos = self.cos.index_select(0, pos)
                sin = self.sin.index_select(0, pos)
                keys = torch.arange(self.max_len, device=self.device)
                # additive form once per forward (a boolean mask is converted by every attention call)
                mask = torch.zeros((pos.shape[0], self.max_len), dtype=cd, device=self.device).masked_fill_(
                    keys[None, :] > pos[:, None], float("-inf"))
                made.append((cos, sin, mask))
            return made[0]

        for block, kv in zip(self.blocks, cache):
            x = block.forward(x, rows, kv, pos, tables=(self.cos, self.sin), oob_flag=self._pos_oob)
        if last_only:
            x = x[:, -1:, :]
        return self.token_embedding(self.final_norm(x), reverse=True)

    def _weights_fingerprint(self):
        """Changes whenever a variable is assigned, replaced or written in place."""
        fp = []
        for layer in self._flatten_layers(include_self=True):
            for v in layer._variables:
                t = v.value
                fp.append((id(v), v.version, t.data_ptr(), t._version))
        return hash(tuple(fp))

    def _session(self, batch):
        """Static buffers for `batch` sequences (KV cache, token, position, output), the
        decode-step graph and one prompt graph per prompt length; dropped when a weight
        changes (the graphs hold the addresses of the layers' derived copies)."""
        fp = self._weights_fingerprint()
        if self._graphs.get("weights") != fp:
            self._graphs = {"weights": fp}
        sess = self._graphs.get(batch)
        if sess is None:
            dev = self.device
            sess = dict(
                cache=self.new_cache(batch),
                out=torch.zeros((batch, self.max_len), dtype=torch.int64, device=dev),
                tok=torch.zeros((batch, 1), dtype=torch.int64, device=dev),
                pos=torch.zeros((1,), dtype=torch.int64, device=dev),
                idx=torch.zeros((1,), dtype=torch.int64, device=dev),
                stream=torch.cuda.Stream(dev), step_graph=None, prompts={})
            self._graphs[batch] = sess
        return sess

    def _graphed_generate(self, prompt, steps, stats):
        B, P = prompt.shape
        sess = self._session(B)
        cache, out_buf, tok_buf, pos_buf, idx_buf = (sess[k] for k in ("cache", "out", "tok", "pos", "idx"))
        cur = torch.cuda.current_stream(self.device)

        def prefill(ids):
            # stale cache rows beyond the current position are never attended (the mask keeps
            # keys <= pos), so the static cache needs no clearing between sequences
            logits = self.forward(ids, torch.arange(P, device=self.device), cache)
            token = logits[:, -1, :].argmax(dim=-1, keepdim=True)
            out_buf[:, :1] = token
            tok_buf.copy_(token)
            pos_buf.fill_(P)
            idx_buf.fill_(1)

        def step():
            lg = self.forward(tok_buf, pos_buf, cache)
            nxt = lg[:, -1, :].argmax(dim=-1, keepdim=True)
            out_buf.index_copy_(1, idx_buf, nxt)
            tok_buf.copy_(nxt)
            pos_buf.add_(1)
            idx_buf.add_(1)

        def capture(fn):
            # one eager run first (first-call set-up, scratch and derived copies), then the capture
            side = sess["stream"]
            side.wait_stream(cur)
            with torch.cuda.stream(side):
                fn()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    fn()
            cur.wait_stream(side)
            return graph

        entry = sess["prompts"].get(P)
        if entry is None:
            ids = torch.zeros((B, P), dtype=torch.int64, device=self.device)
            ids.copy_(prompt)
            entry = sess["prompts"][P] = (ids, capture(lambda: prefill(ids)))
        ids, prompt_graph = entry
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        ev[0].record()
        ids.copy_(prompt)
        prompt_graph.replay()
        ev[1].record()
        done = 1
        if sess["step_graph"] is None and steps > 2:
            # (the eager run inside capture() is a real step of this sequence)
            sess["step_graph"] = capture(step)
            done += 1
        ev[2].record()
        timed = steps - done
        for _ in range(timed):
            if sess["step_graph"] is not None:
                sess["step_graph"].replay()
            else:
                step()
        ev[3].record()
        result = out_buf[:, :steps].clone()
        if stats is not None:
            torch.cuda.synchronize(self.device)
            stats.update(prefill_ms=ev[0].elapsed_time(ev[1]), decode_ms=ev[2].elapsed_time(ev[3]),
                         decode_steps=timed, batch=B)
        self.check_positions()
        return result

    def generate(self, prompt, steps, use_graph=True, stats=None):
        """Greedy decode: prompt [B, P] -> generated ids [B, steps].  The prompt is one
        forward over P positions; each later step is one forward over one position that also
        feeds its token back.  With use_graph both are replayed from HIP graphs (shapes and
        buffers are static, the position lives on the device) that the model keeps per batch
        size and prompt length: the first call for a shape captures them (untimed), later
        calls only replay.  `stats` (a dict) receives prefill_ms, decode_ms, decode_steps as
        measured with device events."""
        prompt = prompt.to(self.device)
        B, P = prompt.shape
        if P + steps > self.max_len:
            raise ValueError(f"prompt {P} + steps {steps} exceeds max_len {self.max_len}")
        if use_graph:
            return self._graphed_generate(prompt, steps, stats)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        cache = self.new_cache(B)
        ev[0].record()
        logits = self.forward(prompt, torch.arange(P, device=self.device), cache)
        token = logits[:, -1, :].argmax(dim=-1)
        ev[1].record()
        out_buf = torch.zeros((B, steps), dtype=torch.int64, device=self.device)
        out_buf[:, 0] = token
        tok_buf = token.clone().reshape(B, 1)
        pos_buf = torch.full((1,), P, dtype=torch.int64, device=self.device)
        idx_buf = torch.ones((1,), dtype=torch.int64, device=self.device)

        def step():
            lg = self.forward(tok_buf, pos_buf, cache)
            nxt = lg[:, -1, :].argmax(dim=-1, keepdim=True)
            out_buf.index_copy_(1, idx_buf, nxt)
            tok_buf.copy_(nxt)
            pos_buf.add_(1)
            idx_buf.add_(1)

        done = 1
        ev[2].record()
        timed = steps - done
        for _ in range(timed):
            step()
        ev[3].record()
        if stats is not None:
            torch.cuda.synchronize(self.device)
            stats.update(prefill_ms=ev[0].elapsed_time(ev[1]), decode_ms=ev[2].elapsed_time(ev[3]),
                         decode_steps=timed, batch=B)
        self.check_positions()
        return out_buf
