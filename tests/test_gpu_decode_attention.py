"""GPU: the one-position attention kernel of the decoder harness against the torch ops it
replaces (rotation, cache update, masked scaled-dot-product attention)."""

import pytest
import torch

from keras_amd import ops as kops
from keras_amd.decoder_harness import apply_rope, rope_tables

pytestmark = pytest.mark.gpu


def torch_step(q, k, v, cos_t, sin_t, pos, kc, vc):
    """The harness's own op sequence for one position (decoder_harness.DecoderBlock.forward)."""
    cos, sin = cos_t.index_select(0, pos), sin_t.index_select(0, pos)
    H = q.shape[2]
    qk = apply_rope(torch.cat((q, k), dim=2), cos, sin)
    qr, kr = qk[:, :, :H], qk[:, :, H:]
    kc.index_copy_(2, pos, kr.transpose(1, 2))
    vc.index_copy_(2, pos, v.transpose(1, 2))
    keys = torch.arange(kc.shape[2], device=q.device)
    mask = torch.zeros((1, kc.shape[2]), dtype=q.dtype, device=q.device).masked_fill_(
        keys[None, :] > pos[:, None], float("-inf"))
    a = torch.nn.functional.scaled_dot_product_attention(qr.transpose(1, 2), kc, vc, attn_mask=mask[None, None])
    return a.transpose(1, 2)


def exact_step(q, k, v, cos_t, sin_t, pos, kc, vc):
    """float64 attention over the bfloat16 cache as the kernel leaves it."""
    p = int(pos.item())
    cos, sin = cos_t[p].double(), sin_t[p].double()
    half = q.shape[-1] // 2
    rot = lambda x: (x.double() * cos).to(torch.bfloat16).double() + \
        (torch.cat((x[..., half:], x[..., :half]), -1).double() * sin).to(torch.bfloat16).double()
    qr = rot(q).to(torch.bfloat16).double()[:, 0]                       # [B, H, hd]
    K, V = kc[:, :, : p + 1].double(), vc[:, :, : p + 1].double()       # [B, H, n, hd]
    s = torch.einsum("bhd,bhnd->bhn", qr, K) / (q.shape[-1] ** 0.5)
    return torch.einsum("bhn,bhnd->bhd", torch.softmax(s, -1), V)[:, None]


@pytest.mark.parametrize("B,H,max_len,pos", [(1, 32, 256, 0), (1, 32, 256, 130), (8, 32, 256, 255),
                                             (2, 5, 64, 17), (3, 8, 1024, 1000), (1, 32, 4096, 4095),
                                             (1, 2, 20000, 19999)])
def test_decode_attention_matches_torch_ops(dev, B, H, max_len, pos):
    g = torch.Generator().manual_seed(B * 1000 + pos)
    hd = 128
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = mk(B, 1, H, hd), mk(B, 1, H, hd), mk(B, 1, H, hd)
    kc0, vc0 = mk(B, H, max_len, hd), mk(B, H, max_len, hd)
    cos_t, sin_t = rope_tables(hd, max_len, dev, dtype=torch.bfloat16)
    pos_t = torch.tensor([pos], dtype=torch.int64, device=dev)
    kc_a, vc_a, kc_b, vc_b = kc0.clone(), vc0.clone(), kc0.clone(), vc0.clone()
    want = torch_step(q, k, v, cos_t, sin_t, pos_t, kc_a, vc_a)
    assert kops.decode_attention_supported(q, kc_b)
    got = kops.decode_attention(q, k, v, cos_t, sin_t, pos_t, kc_b, vc_b)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (B, 1, H, hd)
    # the caches: the new rows are the torch ops' rows bit for bit, every other row untouched
    assert torch.equal(kc_a.view(torch.int16), kc_b.view(torch.int16))
    assert torch.equal(vc_a.view(torch.int16), vc_b.view(torch.int16))
    exact = exact_step(q, k, v, cos_t, sin_t, pos_t, kc_b, vc_b)
    denom = exact.abs().max().item()
    err_kernel = (got.double() - exact).abs().max().item() / denom
    err_torch = (want.double() - exact).abs().max().item() / denom
    # one bfloat16 rounding of the result: half an ulp of the largest magnitudes
    assert err_kernel <= 4e-3, (err_kernel, err_torch)
    assert err_kernel <= 2 * err_torch + 1e-3


def test_decode_attention_position_is_read_on_the_device(dev):
    # a HIP graph captured once replays with whatever position the device tensor then holds
    g = torch.Generator().manual_seed(4)
    B, H, hd, max_len = 2, 4, 128, 64
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = mk(B, 1, H, hd), mk(B, 1, H, hd), mk(B, 1, H, hd)
    kc, vc = mk(B, H, max_len, hd), mk(B, H, max_len, hd)
    cos_t, sin_t = rope_tables(hd, max_len, dev, dtype=torch.bfloat16)
    pos_t = torch.zeros(1, dtype=torch.int64, device=dev)
    out = torch.empty(B, 1, H, hd, dtype=torch.bfloat16, device=dev)
    side = torch.cuda.Stream()
    kc_g, vc_g = kc.clone(), vc.clone()
    with torch.cuda.stream(side):
        kops.decode_attention(q, k, v, cos_t, sin_t, pos_t, kc_g, vc_g)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out.copy_(kops.decode_attention(q, k, v, cos_t, sin_t, pos_t, kc_g, vc_g))
    torch.cuda.synchronize()
    for p in (5, 40, 6, 63):
        kc_g.copy_(kc)
        vc_g.copy_(vc)
        pos_t.fill_(p)
        graph.replay()
        torch.cuda.synchronize()
        kc_e, vc_e = kc.clone(), vc.clone()
        eager = kops.decode_attention(q, k, v, cos_t, sin_t, pos_t, kc_e, vc_e)
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), p
        assert torch.equal(kc_g.view(torch.int16), kc_e.view(torch.int16))


def test_decode_attention_rejects(dev):
    hd = 128
    z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt, device=dev)
    cos_t, sin_t = rope_tables(hd, 16, dev, dtype=torch.bfloat16)
    pos = torch.zeros(1, dtype=torch.int64, device=dev)
    q = z(1, 1, 2, hd)
    with pytest.raises(ValueError):
        kops.decode_attention(z(1, 2, 2, hd), z(1, 2, 2, hd), z(1, 2, 2, hd), cos_t, sin_t, pos,
                              z(1, 2, 16, hd), z(1, 2, 16, hd))
    with pytest.raises(ValueError):
        kops.decode_attention(q, q, q, cos_t, sin_t, pos, z(1, 2, 8, hd), z(1, 2, 8, hd))
    with pytest.raises(ValueError):
        kops.decode_attention(q, q, q, cos_t, sin_t, pos.to(torch.int32), z(1, 2, 16, hd), z(1, 2, 16, hd))
    with pytest.raises(TypeError):
        kops.decode_attention(q.float(), q.float(), q.float(), cos_t, sin_t, pos,
                              z(1, 2, 16, hd), z(1, 2, 16, hd))
    assert not kops.decode_attention_supported(z(1, 1, 2, 64), z(1, 2, 16, 64))


@pytest.mark.parametrize("rows,dim", [(1, 4096), (8, 4096), (3, 128), (2, 8192), (5, 2056)])
def test_rmsnorm_matches_torch(dev, rows, dim):
    g = torch.Generator().manual_seed(rows + dim)
    x = (torch.randn(rows, 1, dim, generator=g) * 3).to(torch.bfloat16).to(dev)
    w = (torch.rand(dim, generator=g) + 0.5).to(torch.bfloat16).to(dev)
    assert kops.rmsnorm_supported(x, w)
    got = kops.rmsnorm(x, w, 1e-6)
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    exact = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    want = torch.nn.functional.rms_norm(x, (dim,), w, 1e-6)
    # one rounding of the float32 result: within one bfloat16 ulp of the exact value, and as
    # close to it as torch's own kernel
    rel = lambda a: ((a.double() - exact).abs() / exact.abs().clamp_min(1e-3)).max().item()
    assert rel(got) <= 2 ** -8 and rel(got) <= rel(want) + 2 ** -9
    # rows given by a stride (a column slice of a wider tensor)
    wide = torch.randn(rows, dim + 64, generator=g).to(torch.bfloat16).to(dev)
    assert torch.equal(kops.rmsnorm(wide[:, :dim], w, 1e-6).view(torch.int16),
                       kops.rmsnorm(wide[:, :dim].contiguous(), w, 1e-6).view(torch.int16))


@pytest.mark.parametrize("rows,dim", [(1, 14336), (8, 14336), (3, 64), (2, 11008)])
def test_silu_mul_matches_torch(dev, rows, dim):
    g = torch.Generator().manual_seed(rows * 7 + dim)
    both = (torch.randn(rows, 2 * dim, generator=g) * 2).to(torch.bfloat16).to(dev)
    gate, up = both[:, :dim], both[:, dim:]          # column slices: rows by stride
    assert kops.silu_mul_supported(gate, up)
    got = kops.silu_mul(gate, up)
    want = torch.nn.functional.silu(gate) * up
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    # the same two roundings; exp may differ in its last float32 bit, which moves a rounding
    # of silu(g) by one bfloat16 ulp on a few elements at most
    diff = (got.float() - want.float()).abs()
    assert (diff <= want.float().abs() * 2 ** -7 + 1e-30).all()
    assert (diff > 0).float().mean().item() < 0.01
    assert torch.equal(kops.silu_mul(gate.contiguous(), up.contiguous()).view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("bad", [-1, 16, 1 << 40])
def test_decode_attention_position_outside_the_cache(dev, bad):
    # where the torch ops (index_copy_ into the caches) raise, the kernel writes nothing to the
    # caches, returns zero rows and raises the caller's flag; without a flag the call raises itself
    hd, max_len = 128, 16
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(dev)
    cos_t, sin_t = rope_tables(hd, max_len, dev, dtype=torch.bfloat16)
    q, k, v = r(2, 1, 4, hd), r(2, 1, 4, hd), r(2, 1, 4, hd)
    kc, vc = r(2, 4, max_len, hd), r(2, 4, max_len, hd)
    kc0, vc0 = kc.clone(), vc.clone()
    pos = torch.full((1,), bad, dtype=torch.int64, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    out = kops.decode_attention(q, k, v, cos_t, sin_t, pos, kc, vc, oob_flag=flag)
    torch.cuda.synchronize()
    assert flag.item() == 1 and out.abs().max().item() == 0
    assert torch.equal(kc.view(torch.int16), kc0.view(torch.int16))
    assert torch.equal(vc.view(torch.int16), vc0.view(torch.int16))
    with pytest.raises(IndexError):
        kops.decode_attention(q, k, v, cos_t, sin_t, pos, kc, vc)
    # a position inside leaves a raised flag alone and a clear one clear
    pos.fill_(max_len - 1)
    flag.zero_()
    kops.decode_attention(q, k, v, cos_t, sin_t, pos, kc, vc, oob_flag=flag)
    assert flag.item() == 0
    assert not torch.equal(kc.view(torch.int16), kc0.view(torch.int16))
