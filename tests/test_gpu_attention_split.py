"""Attention with a head's positions dealt to several workgroups, and the output projection that
combines the slices' results while it stages its row (MI355X only).

Floating point: the split path rounds every slice's result to fp16 before the slices are combined,
so it differs from the one-workgroup-per-head kernel by those roundings; the bound used here is
rel-L2 <= 2e-3 (measured 4e-4).  Slice s of S takes the blocks of 64 positions s, s + S, ...; wherever
only one slice holds positions (one slice asked for, or a position below 64) the combined result
must equal the unsplit kernel's bit for bit.
The output projection's staging must equal the combine kernel followed by the plain projection bit
for bit (same arithmetic on the same operands), and the C oracle's fused product within 1e-3.
"""
import math
import sys

import numpy as np
import pytest
import torch

from oracle import cherryq_oracle as orc
from oracle import c_oracle

pytestmark = pytest.mark.gpu

SPLIT_TOL = 2e-3
NAMES = ("cherry_indices", "cherry_weight", "qweight", "scales")


@pytest.fixture(scope="module")
def dec():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cherryq_decoder
    return cherryq_decoder


def stream():
    return torch.cuda.current_stream().cuda_stream


def rel(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm())


def announce(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("nh,nkv,ml,steps", [(8, 4, 64, 20), (4, 4, 600, 530), (32, 32, 256, 256), (8, 2, 200, 200)])
def test_split_attention_matches_the_unsplit_kernel_over_a_growing_cache(dec, nh, nkv, ml, steps):
    announce("split attention growing cache", nh, nkv, ml, steps)
    lib = dec._lib
    torch.manual_seed(5)
    hd = 128
    caches = {s: (torch.zeros(nkv, ml, hd, device="cuda").half(), torch.zeros(nkv, ml, hd, device="cuda").half())
              for s in (0, 1, 2, 4, 8)}
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    worst = 0.0
    for step in range(steps):
        q = torch.randn(1, nh * hd, device="cuda").half()
        k = torch.randn(1, nkv * hd, device="cuda").half()
        v = torch.randn(1, nkv * hd, device="cuda").half()
        want = torch.empty_like(q)
        assert lib.cherryq_decode_rope_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), caches[0][0].data_ptr(),
                                                     caches[0][1].data_ptr(), want.data_ptr(), pos.data_ptr(), nh, nkv, hd,
                                                     ml, 10000.0, stream()) == 0
        got = {}
        for s in (1, 2, 4, 8):
            part = torch.full((s, nh * hd), float("nan"), dtype=torch.float16, device="cuda")
            msum = torch.full((s, nh, 2), float("nan"), dtype=torch.float32, device="cuda")
            dec.rope_attention_split(q, k, v, caches[s][0], caches[s][1], part, msum, pos, nh, nkv, hd, ml, 10000.0, slices=s)
            out = torch.empty_like(q)
            dec.attention_combine(part, msum, out)
            got[s] = out
        if step % 23 == 0 or step == steps - 1 or step in (63, 64, 65, 127, 128):
            torch.cuda.synchronize()
            assert torch.equal(got[1], want), ("one slice", step)
            for s in (2, 4, 8):
                assert torch.isfinite(got[s]).all(), (s, step)
                if step < 64:   # every position lies in the first slice
                    assert torch.equal(got[s], want), (s, step)
                else:
                    r = rel(got[s], want)
                    worst = max(worst, r)
                    assert r <= SPLIT_TOL, (s, step, r)
        pos.add_(1)
    torch.cuda.synchronize()
    for s in (1, 2, 4, 8):
        assert torch.equal(caches[s][0], caches[0][0]) and torch.equal(caches[s][1], caches[0][1]), s
    print("worst rel-L2 split vs unsplit: %.2e" % worst, flush=True)


def test_split_attention_against_a_float64_softmax(dec):
    """Independent of the unsplit kernel: rotary embedding, scores, softmax and the weighted sum of the
    value rows restated in torch float64 from the cache the kernel itself filled."""
    announce("split attention vs float64")
    torch.manual_seed(6)
    nh, nkv, hd, ml = 8, 4, 128, 256
    kc = torch.zeros(nkv, ml, hd, device="cuda").half()
    vc = torch.zeros_like(kc)
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, device="cuda").float() / hd))

    def rope(x, p):   # x (heads, hd) fp16 -> rotated, float64 arithmetic on the fp16 cos / sin the reference caches
        ang = p * inv_freq
        cos = torch.cat([ang.cos(), ang.cos()]).half().double()
        sin = torch.cat([ang.sin(), ang.sin()]).half().double()
        xd = x.double()
        rot = torch.cat([-xd[:, hd // 2:], xd[:, :hd // 2]], dim=1)
        return xd * cos + rot * sin

    for p in range(200):
        q = torch.randn(1, nh * hd, device="cuda").half()
        k = torch.randn(1, nkv * hd, device="cuda").half()
        v = torch.randn(1, nkv * hd, device="cuda").half()
        part = torch.empty(4, nh * hd, dtype=torch.float16, device="cuda")
        msum = torch.empty(4, nh, 2, dtype=torch.float32, device="cuda")
        dec.rope_attention_split(q, k, v, kc, vc, part, msum, pos, nh, nkv, hd, ml, 10000.0)
        out = torch.empty_like(q)
        dec.attention_combine(part, msum, out)
        if p in (0, 1, 63, 64, 100, 128, 199):
            torch.cuda.synchronize()
            qr = rope(q.view(nh, hd), p)
            K = kc[:, :p + 1].double().repeat_interleave(nh // nkv, dim=0)
            V = vc[:, :p + 1].double().repeat_interleave(nh // nkv, dim=0)
            att = torch.softmax(torch.einsum("hd,hjd->hj", qr, K) / math.sqrt(hd), -1)
            want = torch.einsum("hj,hjd->hd", att, V).reshape(1, -1)
            assert rel(out, want) < 5e-3, p
            # the slices' sums of exponentials add up to the softmax denominator
            m, l = msum[..., 0].double(), msum[..., 1].double()
            big = m.max(0).values
            denom = (torch.exp(m - big) * l).sum(0)
            sc = torch.einsum("hd,hjd->hj", qr, K) / math.sqrt(hd)
            want_denom = torch.exp(sc - sc.max(-1, keepdim=True).values).sum(-1)
            ratio = denom * torch.exp(big - sc.max(-1).values) / want_denom
            assert float((ratio - 1).abs().max()) < 5e-3, p
        pos.add_(1)


def test_split_attention_position_guards_and_rejections(dec):
    announce("split attention guards")
    lib = dec._lib
    nh, nkv, hd, ml = 4, 2, 128, 96
    torch.manual_seed(7)
    q = torch.randn(1, nh * hd, device="cuda").half()
    k = torch.randn(1, nkv * hd, device="cuda").half()
    v = torch.randn(1, nkv * hd, device="cuda").half()
    for bad in (ml, ml + 7, -1, -(2 ** 31)):
        kc = torch.randn(nkv, ml, hd, device="cuda").half()
        vc = torch.randn(nkv, ml, hd, device="cuda").half()
        kc0, vc0 = kc.clone(), vc.clone()
        pos = torch.tensor([bad], dtype=torch.int32, device="cuda")
        part = torch.zeros(4, nh * hd, dtype=torch.float16, device="cuda")
        msum = torch.zeros(4, nh, 2, dtype=torch.float32, device="cuda")
        dec.rope_attention_split(q, k, v, kc, vc, part, msum, pos, nh, nkv, hd, ml, 10000.0)
        out = torch.zeros_like(q)
        dec.attention_combine(part, msum, out)
        torch.cuda.synchronize()
        assert torch.equal(kc, kc0) and torch.equal(vc, vc0), bad
        assert torch.isnan(out).all(), bad
    # the last valid position works; empty slices leave (-inf, 0) and zeros
    kc = torch.randn(nkv, ml, hd, device="cuda").half()
    vc = torch.randn(nkv, ml, hd, device="cuda").half()
    pos = torch.tensor([ml - 1], dtype=torch.int32, device="cuda")
    part = torch.full((4, nh * hd), float("nan"), dtype=torch.float16, device="cuda")
    msum = torch.full((4, nh, 2), float("nan"), dtype=torch.float32, device="cuda")
    dec.rope_attention_split(q, k, v, kc, vc, part, msum, pos, nh, nkv, hd, ml, 10000.0)
    out = torch.zeros_like(q)
    dec.attention_combine(part, msum, out)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    # positions 0 .. 95 are blocks 0 and 1: slices 2 and 3 hold nothing
    assert torch.equal(part[2:], torch.zeros_like(part[2:]))
    assert torch.isneginf(msum[2:, :, 0]).all() and (msum[2:, :, 1] == 0).all()
    assert (msum[:2, :, 1] >= 1).all()
    # argument checks of the C ABI
    p = [q.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(), part.data_ptr(), msum.data_ptr()]
    assert lib.cherryq_decode_attention_max_slices() == 8 and lib.cherryq_decode_attention_projection_slices() == 4
    assert lib.cherryq_decode_rope_attention_split_f16(*p, 9, pos.data_ptr(), nh, nkv, hd, ml, 10000.0, stream()) != 0
    assert lib.cherryq_decode_rope_attention_split_f16(*p, 0, pos.data_ptr(), nh, nkv, hd, ml, 10000.0, stream()) != 0
    assert lib.cherryq_decode_rope_attention_split_f16(*p, 4, pos.data_ptr(), nh, nkv, 64, ml, 10000.0, stream()) != 0
    assert lib.cherryq_decode_rope_attention_split_f16(*p, 4, pos.data_ptr(), nh, 3, hd, ml, 10000.0, stream()) != 0
    assert lib.cherryq_decode_rope_attention_split_f16(*p, 4, None, nh, nkv, hd, ml, 10000.0, stream()) != 0
    assert lib.cherryq_decode_rope_attention_split_f16(*p, 4, pos.data_ptr(), nh, nkv, hd, 10 ** 6, 10000.0, stream()) != 0
    assert lib.cherryq_decode_attention_combine_f16(part.data_ptr(), msum.data_ptr(), 9, out.data_ptr(), nh, hd, stream()) != 0
    assert lib.cherryq_decode_attention_combine_f16(part.data_ptr(), msum.data_ptr(), 4, out.data_ptr(), nh, 64, stream()) != 0
    torch.cuda.synchronize()


# output projections: one tile per compute unit (4096 -> 4096), two and three teams (4096 -> 8192, -> 11008),
# walking tiles (4096 -> 16384), 64 units per column (8192 -> 8192), a short ragged layer
OUT_SHAPES = [(4, 4096, 4096), (3, 4096, 4096), (4, 4096, 8192), (3, 4096, 11008), (4, 4096, 16384), (3, 4096, 16384),
              (4, 8192, 8192), (3, 8192, 8192), (4, 1024, 264), (3, 2304, 4104)]


@pytest.mark.parametrize("bits,k,n", OUT_SHAPES)
def test_output_projection_combines_the_slices_like_the_combine_kernel(dec, bits, k, n):
    announce("attention out projection", bits, k, n)
    gen = torch.Generator(device="cuda").manual_seed(41 + bits + k)
    cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=1 / 256)
    m = dec.random_packed_linear(cfg, k, n, gen, "cuda")
    p = {b: getattr(m, b).cpu().numpy() for b in NAMES}
    assert m.prepack()
    assert dec.matvec_attention_prepacked_supported(m)
    heads = k // 128
    rng = np.random.default_rng(23 + k)
    part = torch.from_numpy(rng.standard_normal((4, k)).astype(np.float16)).cuda()
    mx = rng.standard_normal((4, heads)).astype(np.float32) * 3
    sm = (1 + rng.random((4, heads)) * 60).astype(np.float32)
    # empty slices (as the attention kernel leaves them) on some heads, every combination of the last three
    for h in range(heads):
        for s in range(1, 4):
            if (h >> (s - 1)) & 1 and h % 3 == 0:
                mx[s, h], sm[s, h] = -np.inf, 0.0
                part[s, 128 * h:128 * (h + 1)] = 0
    msum = torch.from_numpy(np.stack([mx, sm], axis=-1)).cuda().contiguous()
    row = torch.empty(1, k, dtype=torch.float16, device="cuda")
    dec.attention_combine(part, msum, row)
    torch.cuda.synchronize()
    # the combine kernel against float64
    md, ld, pd = torch.from_numpy(mx).double(), torch.from_numpy(sm).double(), part.cpu().double()
    w = torch.exp(md - md.max(0).values) * ld
    c = (w / w.sum(0)).repeat_interleave(128, dim=1)
    assert rel(row.cpu(), (c * pd).sum(0, keepdim=True)) < 1e-3
    for accumulate in (False, True):
        base = torch.from_numpy(rng.standard_normal((1, n)).astype(np.float16)).cuda()
        want, got = base.clone(), base.clone()
        dec.matvec_group_prepacked([m], row, [want], accumulate=accumulate)
        dec.matvec_attention_prepacked(m, part, msum, got, accumulate=accumulate)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), (accumulate, rel(got, want))
    ref = c_oracle.fused(row.cpu().numpy(), p, bits, 128)
    out = torch.empty(1, n, dtype=torch.float16, device="cuda")
    dec.matvec_attention_prepacked(m, part, msum, out)
    torch.cuda.synchronize()
    assert orc.rel_l2(out.cpu().numpy(), ref) <= 1e-3


def test_output_projection_rejections(dec):
    announce("attention out projection rejections")
    lib = dec._lib
    gen = torch.Generator(device="cuda").manual_seed(3)
    cfg = dec.DecoderConfig(w_bits=4, group_size=128, cherry_fraction=1 / 256)
    # 11008 input channels run on a deeper launch geometry that has no combining prologue
    assert lib.cherryq_decode_matvec_attention_prepacked_supported(4, 11008, 4096, 40) == 0
    assert lib.cherryq_decode_matvec_attention_prepacked_supported(4, 4096, 4096, 16) == 1
    assert lib.cherryq_decode_matvec_attention_prepacked_supported(4, 4032, 4096, 16) == 0   # not whole heads
    assert lib.cherryq_decode_matvec_attention_prepacked_supported(5, 4096, 4096, 16) == 0
    m = dec.random_packed_linear(cfg, 1024, 256, gen, "cuda")
    assert m.prepack()
    st = m._stream
    part = torch.zeros(4, 1024, dtype=torch.float16, device="cuda")
    msum = torch.zeros(4, 8, 2, dtype=torch.float32, device="cuda")
    out = torch.zeros(1, 256, dtype=torch.float16, device="cuda")
    args = lambda **kw: [kw.get("bits", 4), kw.get("part", part.data_ptr()), kw.get("ml", msum.data_ptr()), kw.get("slices", 4),
                         st.data_ptr(), kw.get("bytes", st.numel()), out.data_ptr(), kw.get("k", 1024), 256, m.num_cherries, 0,
                         stream()]
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args()) == 0
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args(slices=2)) != 0
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args(part=None)) != 0
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args(ml=None)) != 0
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args(bytes=st.numel() - 256)) != 0
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args(part=part.data_ptr() + 2)) != 0
    assert lib.cherryq_decode_matvec_attention_prepacked_f16(*args(bits=2)) != 0
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        dec.matvec_attention_prepacked(m, part[:2].contiguous(), msum, out)
    m2 = dec.random_packed_linear(cfg, 1024, 256, gen, "cuda")
    with pytest.raises(RuntimeError):
        dec.matvec_attention_prepacked(m2, part, msum, out)   # not repacked


@pytest.mark.parametrize("max_len,setting", [(256, True), (1024, None)])
def test_decoder_token_steps_with_and_without_split_attention(dec, max_len, setting):
    """The same small decoder, layers repacked, with attention dealt to four workgroups per head +
    combining o_proj (forced on a 256-position cache; chosen by the decoder itself for 1024
    positions, where only the rows up to the position are read), and with one workgroup per head +
    plain o_proj: logits under teacher forcing agree within the split path's rounding, eager and as
    graph replays (replayed twice with unrelated work in between), and both agree with the
    dense-weight torch restatement."""
    announce("decoder split attention on / off", max_len, setting)
    cfg = dec.DecoderConfig(hidden_size=1024, intermediate_size=2816, num_hidden_layers=3, num_attention_heads=8,
                            num_key_value_heads=8, vocab_size=2048, max_position_embeddings=max_len, w_bits=4)
    d = dec.CherryLlamaDecoder(cfg, seed=11)
    assert d.split_attn is None
    assert d.prepack(only_recommended=False) == 7 * cfg.num_hidden_layers
    assert dec.matvec_attention_prepacked_supported(d.layers[0].o_proj)
    ids = (torch.arange(150) * 37 + 5) % cfg.vocab_size
    want = d.reference_logits(ids)
    d.split_attn = False
    plain = d.step_logits(ids)
    d.split_attn = setting
    d._graph = None
    eager = d.step_logits(ids)
    graph = d.step_logits(ids, use_graph=True)
    _ = d.reference_logits(ids[:4])
    graph2 = d.step_logits(ids, use_graph=True)
    assert torch.equal(graph, eager) and torch.equal(graph2, eager)
    assert not torch.equal(eager[100], plain[100])   # the split path really ran (positions beyond the first block)
    assert torch.equal(eager[:64], plain[:64])       # below 64 positions one slice holds everything
    for i in (64, 65, 100, 128, 149):
        assert rel(eager[i], plain[i]) < 5e-3, i
        assert rel(eager[i], want[i]) < 2e-2, i
