"""Decode-step glue kernels and the 7B-shaped decoder built from them (MI355X only)."""
import ctypes
import math
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dec():
    assert torch.cuda.is_available()
    import cherryq_decoder
    return cherryq_decoder


def rel(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm())


def stream():
    return torch.cuda.current_stream().cuda_stream


def test_add_rmsnorm_kernel(dec):
    print("[case] add_rmsnorm", flush=True)
    lib = dec._lib
    torch.manual_seed(0)
    for H in (4096, 256, 5120):
        h = torch.randn(1, H, device="cuda").half()
        d = torch.randn(1, H, device="cuda").half()
        w = (torch.rand(H, device="cuda") + 0.5).half()
        y = torch.empty_like(h)
        h2 = h.clone()
        assert lib.cherryq_decode_add_rmsnorm_f16(h2.data_ptr(), d.data_ptr(), w.data_ptr(), y.data_ptr(), H, 1e-6,
                                                  stream()) == 0
        torch.cuda.synchronize()
        hs = h + d
        xf = hs.float()
        want = w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).half()
        assert torch.equal(h2, hs)
        assert rel(y, want) < 1e-3
        h3 = h.clone()
        assert lib.cherryq_decode_add_rmsnorm_f16(h3.data_ptr(), None, w.data_ptr(), y.data_ptr(), H, 1e-6, stream()) == 0
        torch.cuda.synchronize()
        assert torch.equal(h3, h)


def test_rope_cache_and_attention_kernels(dec):
    print("[case] rope/attention", flush=True)
    lib = dec._lib
    torch.manual_seed(1)
    nh, nkv, hd, ml = 8, 4, 128, 64
    kc = torch.zeros(nkv, ml, hd, device="cuda").half()
    vc = torch.zeros_like(kc)
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, device="cuda").float() / hd))

    def rope(x, p):
        fr = p * inv
        emb = torch.cat([fr, fr])
        c, s = emb.cos().half(), emb.sin().half()
        x1, x2 = x[..., :hd // 2], x[..., hd // 2:]
        return x * c + torch.cat([-x2, x1], -1) * s

    ks, vs = [], []
    for p in range(20):
        q = torch.randn(nh, hd, device="cuda").half()
        k = torch.randn(nkv, hd, device="cuda").half()
        v = torch.randn(nkv, hd, device="cuda").half()
        pos.fill_(p)
        q2 = q.clone()
        assert lib.cherryq_decode_rope_cache_f16(q2.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                                 pos.data_ptr(), nh, nkv, hd, ml, 10000.0, stream()) == 0
        out = torch.empty(nh, hd, device="cuda").half()
        assert lib.cherryq_decode_attention_f16(q2.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(),
                                                pos.data_ptr(), nh, nkv, hd, ml, stream()) == 0
        torch.cuda.synchronize()
        qr, kr = rope(q, float(p)), rope(k, float(p))
        ks.append(kr)
        vs.append(v)
        assert rel(q2, qr) < 2e-3
        assert rel(kc[:, p], kr) < 2e-3 and torch.equal(vc[:, p], v)
        K = torch.stack(ks, 1).repeat_interleave(nh // nkv, 0).float()   # (nh, p+1, hd)
        V = torch.stack(vs, 1).repeat_interleave(nh // nkv, 0).float()
        att = torch.softmax(torch.einsum("hd,hjd->hj", qr.float(), K) / math.sqrt(hd), -1)
        want = torch.einsum("hj,hjd->hd", att, V)
        assert rel(out, want) < 5e-3, p


def test_rope_attention_fused_matches_separate_kernels(dec):
    """The one-launch rotary + cache write + attention equals rope_cache followed by attention,
    bit for bit, over a growing cache (grouped-query heads included)."""
    print("[case] rope_attention fused", flush=True)
    lib = dec._lib
    torch.manual_seed(2)
    for nh, nkv, ml, steps in ((8, 4, 64, 20), (4, 4, 600, 530)):
        hd = 128
        kc1 = torch.zeros(nkv, ml, hd, device="cuda").half()
        vc1 = torch.zeros_like(kc1)
        kc2, vc2 = torch.zeros_like(kc1), torch.zeros_like(kc1)
        pos = torch.zeros(1, dtype=torch.int32, device="cuda")
        for step in range(steps):
            q = torch.randn(1, nh * hd, device="cuda").half()
            k = torch.randn(1, nkv * hd, device="cuda").half()
            v = torch.randn(1, nkv * hd, device="cuda").half()
            q1, o1, o2 = q.clone(), torch.empty_like(q), torch.empty_like(q)
            assert lib.cherryq_decode_rope_cache_f16(q1.data_ptr(), k.data_ptr(), v.data_ptr(), kc1.data_ptr(),
                                                     vc1.data_ptr(), pos.data_ptr(), nh, nkv, hd, ml, 10000.0,
                                                     stream()) == 0
            assert lib.cherryq_decode_attention_f16(q1.data_ptr(), kc1.data_ptr(), vc1.data_ptr(), o1.data_ptr(),
                                                    pos.data_ptr(), nh, nkv, hd, ml, stream()) == 0
            assert lib.cherryq_decode_rope_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), kc2.data_ptr(),
                                                         vc2.data_ptr(), o2.data_ptr(), pos.data_ptr(), nh, nkv, hd,
                                                         ml, 10000.0, stream()) == 0
            if step % 37 == 0 or step == steps - 1:
                torch.cuda.synchronize()
                assert rel(o2, o1) < 1e-3, (nh, nkv, step)
            pos.add_(1)
        torch.cuda.synchronize()
        assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)


def test_silu_mul_kernel(dec):
    print("[case] silu_mul", flush=True)
    lib = dec._lib
    g = torch.randn(11008, device="cuda").half() * 3
    u = torch.randn(11008, device="cuda").half()
    o = torch.empty_like(g)
    assert lib.cherryq_decode_silu_mul_f16(g.data_ptr(), u.data_ptr(), o.data_ptr(), 11008, stream()) == 0
    torch.cuda.synchronize()
    assert rel(o, torch.nn.functional.silu(g) * u) < 1e-3


@pytest.mark.parametrize("V,H", [(32000, 4096), (1000, 1024), (517, 512), (32003, 5120), (4099, 8192),
                                 # hidden sizes that are not whole kilobyte pieces per wavefront
                                 (1000, 256), (4099, 384), (517, 8), (2003, 4104), (1000, 6656 + 128), (333, 8184)])
def test_head_kernel_with_fused_final_norm(dec, V, H):
    """fp16 head (final RMSNorm fused or not) against float64 on the same fp16 operands: one
    rounding of the fp32-accumulated sum, rel-L2 below 1e-3; a one-hot row returns the matrix
    column bit for bit; the separate norm launch + this kernel without norm give the same bits."""
    print("[case] head", V, H, flush=True)
    lib = dec._lib
    g = torch.Generator().manual_seed(V + H)
    h = torch.randn(1, H, generator=g).half().cuda()
    nw = (1 + 0.1 * torch.randn(H, generator=g)).half().cuda()
    W = (torch.randn(V, H, generator=g) * 0.02).half().cuda()
    out = torch.full((1, V), float("nan"), dtype=torch.float16, device="cuda")
    for norm in (True, False):
        assert lib.cherryq_decode_head_f16(h.data_ptr(), nw.data_ptr() if norm else None, 1e-6, W.data_ptr(),
                                           out.data_ptr(), V, H, stream()) == 0
        hf = h.float()
        act = (nw.float() * (hf * torch.rsqrt((hf * hf).mean() + 1e-6)).half().float()).half() if norm else h
        want = act.double() @ W.double().t()
        assert rel(out, want) < 1e-3, (norm, rel(out, want))
    onehot = torch.zeros(1, H, dtype=torch.float16, device="cuda")
    onehot[0, H - 3] = 1.0
    assert lib.cherryq_decode_head_f16(onehot.data_ptr(), None, 0.0, W.data_ptr(), out.data_ptr(), V, H, stream()) == 0
    assert torch.equal(out[0], W[:, H - 3])
    normed = torch.empty_like(h)
    h2 = h.clone()
    assert lib.cherryq_decode_add_rmsnorm_f16(h2.data_ptr(), None, nw.data_ptr(), normed.data_ptr(), H, 1e-6, stream()) == 0
    two = torch.empty_like(out)
    assert lib.cherryq_decode_head_f16(normed.data_ptr(), None, 0.0, W.data_ptr(), two.data_ptr(), V, H, stream()) == 0
    assert lib.cherryq_decode_head_f16(h.data_ptr(), nw.data_ptr(), 1e-6, W.data_ptr(), out.data_ptr(), V, H, stream()) == 0
    # the sum of squares is added up in another order than in the separate launch: the normalised
    # row may differ by an fp16 ulp here and there, the logits by a few
    assert rel(out, two.double()) < 1e-3


def test_head_validation(dec):
    lib = dec._lib
    h = torch.zeros(1, 4096, dtype=torch.float16, device="cuda")
    W = torch.zeros(8, 4096, dtype=torch.float16, device="cuda")
    out = torch.zeros(1, 8, dtype=torch.float16, device="cuda")
    assert lib.cherryq_decode_head_supported(32000, 4096) == 1
    assert lib.cherryq_decode_head_supported(32000, 256) == 1 and lib.cherryq_decode_head_supported(32000, 8704) == 0
    assert lib.cherryq_decode_head_supported(32000, 4100) == 0 and lib.cherryq_decode_head_supported(32000, 0) == 0
    assert lib.cherryq_decode_head_f16(None, None, 0.0, W.data_ptr(), out.data_ptr(), 8, 4096, stream()) == -1
    assert lib.cherryq_decode_head_f16(h.data_ptr(), None, 0.0, W.data_ptr(), out.data_ptr(), 0, 4096, stream()) == -2
    assert lib.cherryq_decode_head_f16(h.data_ptr(), None, 0.0, W.data_ptr(), out.data_ptr(), 8, 252, stream()) == -7
    assert lib.cherryq_decode_head_f16(h.data_ptr() + 2, None, 0.0, W.data_ptr(), out.data_ptr(), 8, 4096, stream()) == -6


def test_decode_validation(dec):
    lib = dec._lib
    assert lib.cherryq_decode_add_rmsnorm_f16(None, None, None, None, 4096, 1e-6, None) == -1
    assert lib.cherryq_decode_attention_f16(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, 32, 32, 64, 256, None) == -7
    assert lib.cherryq_decode_attention_f16(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, 32, 5, 128, 256, None) == -2
    assert lib.cherryq_decode_silu_mul_f16(1 << 12, 1 << 12, 1 << 12, 0, None) == -2


@pytest.mark.parametrize("bits", [4, 3])
def test_matvec_group_matches_single_calls(dec, bits):
    """One grouped launch over layers of different widths equals the per-layer entry points
    (which the parity tests pin to the oracle); with a gate vector it equals the per-layer call
    on silu(gate) * up; accumulate adds into the existing output."""
    print("[case] matvec_group", bits, flush=True)
    import quant_cuda
    gen = torch.Generator(device="cuda").manual_seed(5)
    for K, widths, frac in ((1024, (768, 256, 520), 1 / 64), (4096, (4096, 1024, 1024), 1 / 256),
                            (2048, (5504, 5504), 1 / 256), (11008, (4096,), 1 / 256)):
        cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=frac)
        mods = [dec.random_packed_linear(cfg, K, n, gen, "cuda") for n in widths]
        x = torch.randn(1, K, device="cuda", generator=gen).half()
        g = torch.randn(1, K, device="cuda", generator=gen).half()
        want, want_act = [], []
        act = torch.nn.functional.silu(g) * x
        for m in mods:
            for vec, dst in ((x, want), (act, want_act)):
                o = torch.empty(1, m.out_features, dtype=torch.float16, device="cuda")
                quant_cuda.matmul_cherryq(bits, vec, m.qweight, m.cherry_weight, m.cherry_indices, m.scales, o, 128)
                dst.append(o)
        for rep in range(2):  # the second call finds the workspace as the first one left it
            outs = [torch.full((1, n), 7.0, dtype=torch.float16, device="cuda") for n in widths]
            dec.matvec_group(mods, x, outs)
            for o, w in zip(outs, want):
                assert rel(o, w) < 1e-3, (K, widths, rep)
        outs = [torch.full((1, n), 7.0, dtype=torch.float16, device="cuda") for n in widths]
        dec.matvec_group(mods, x, outs, vec_gate=g)
        for o, w in zip(outs, want_act):
            assert rel(o, w) < 1e-3, (K, widths, "gate")
        if K <= 4096:
            # fused RMSNorm: equals the per-layer call on the separately normalised vector
            nw = (torch.rand(K, device="cuda", generator=gen) + 0.5).half()
            h = (torch.randn(1, K, device="cuda", generator=gen) * 3).half()
            y = torch.empty_like(h)
            assert dec._lib.cherryq_decode_add_rmsnorm_f16(h.data_ptr(), None, nw.data_ptr(), y.data_ptr(), K, 1e-6,
                                                           stream()) == 0
            outs = [torch.full((1, n), 7.0, dtype=torch.float16, device="cuda") for n in widths]
            dec.matvec_group(mods, h, outs, norm_weight=nw, eps=1e-6)
            for m, o in zip(mods, outs):
                w = torch.empty_like(o)
                quant_cuda.matmul_cherryq(bits, y, m.qweight, m.cherry_weight, m.cherry_indices, m.scales, w, 128)
                assert rel(o, w) < 1e-3, (K, widths, "norm")
        base = [torch.randn(1, n, device="cuda", generator=gen).half() for n in widths]
        outs = [b.clone() for b in base]
        dec.matvec_group(mods, x, outs, accumulate=True)
        for o, b, w in zip(outs, base, want):
            assert rel(o, (b.float() + w.float())) < 2e-3, (K, widths, "accumulate")
    torch.cuda.synchronize()


def test_matvec_group_validation(dec):
    lib = dec._lib
    assert lib.cherryq_decode_matvec_group_f16(5, None, None, None, 0.0, None, 1, 4096, 16, 128, 0, None, 0, None) == -5
    assert lib.cherryq_decode_matvec_group_f16(4, None, None, None, 0.0, None, 1, 4096, 16, 128, 0, None, 0, None) == -1
    arr = (dec._Layer * 1)(dec._Layer(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, 4096))
    assert lib.cherryq_decode_matvec_group_f16(4, 1 << 12, None, None, 0.0, arr, 5, 4096, 16, 128, 0, 1 << 12, 1 << 20, None) == -2
    assert lib.cherryq_decode_matvec_group_f16(4, 1 << 12, None, None, 0.0, arr, 1, 4096, 16, 128, 0, 1 << 12, 64, None) == -4
    ns = (ctypes.c_int * 2)(4096, 1000)
    assert lib.cherryq_group_workspace_bytes(2, ns) == (4096 + 1024) * 8


@pytest.mark.parametrize("bits", [4, 3])
def test_small_decoder_matches_dense_reference(dec, bits):
    """Two-layer decoder with real packed linears: every variant of the fused token step (grouped
    launches, one launch per operation, forked streams) agrees with the same model on dequantised
    weights and plain torch ops, and its replayed HIP graph equals its eager run bit for bit."""
    print("[case] small decoder", bits, flush=True)
    cfg = dec.DecoderConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                            num_key_value_heads=2, vocab_size=512, max_position_embeddings=32, w_bits=bits,
                            group_size=128, cherry_fraction=1 / 16)
    model = dec.CherryLlamaDecoder(cfg, seed=3)
    ids = torch.randint(0, cfg.vocab_size, (12,), generator=torch.Generator().manual_seed(0))
    want = model.reference_logits(ids)
    for fork, grouped, fuse_norm in ((False, True, True), (False, True, False), (False, False, False),
                                     (True, False, False)):
        model.fuse_norm = fuse_norm
        eager = model.step_logits(ids, use_graph=False, fork=fork, grouped=grouped)
        for t in range(ids.numel()):
            assert rel(eager[t], want[t]) < 2e-2, (t, fork, grouped)
        # several replays with eager work between them, each checked against the eager result
        model._graph = None
        graph = model.step_logits(ids, use_graph=True, fork=fork, grouped=grouped)
        torch.cuda.synchronize()
        _ = model.reference_logits(ids[:4])  # unrelated eager work between replays
        graph2 = model.step_logits(ids, use_graph=True, fork=fork, grouped=grouped)
        assert torch.equal(graph, eager) and torch.equal(graph2, eager), (fork, grouped)
    # every linear repacked into a weight stream: the stream kernels take the grouped launches
    model._graph = None
    model.fuse_norm = True
    assert model.prepack(only_recommended=False) == 14
    for fuse_norm in (True, False):
        model.fuse_norm = fuse_norm
        model._graph = None
        eager = model.step_logits(ids, use_graph=False)
        for t in range(ids.numel()):
            assert rel(eager[t], want[t]) < 2e-2, (t, "prepacked", fuse_norm)
        graph = model.step_logits(ids, use_graph=True)
        _ = model.reference_logits(ids[:4])
        graph2 = model.step_logits(ids, use_graph=True)
        assert torch.equal(graph, eager) and torch.equal(graph2, eager), ("prepacked", fuse_norm)
    # only the weight streams kept (one copy of the weights): the same token step bit for bit, the
    # literal launch sequence and the batched prompt pass go over the streams too
    bytes_before = model.step_bytes()
    kept = eager
    assert model.prepack(only_recommended=False, release_reference=True) == 14
    assert all(m.qweight.numel() == 0 for layer in model.layers for m in layer.children())
    assert model.step_bytes() == bytes_before
    model._graph = None
    assert torch.equal(model.step_logits(ids, use_graph=False), kept)
    assert torch.equal(model.step_logits(ids, use_graph=True), kept)
    literal = model.step_logits(ids, use_graph=False, grouped=False)
    for t in range(ids.numel()):
        assert rel(literal[t], want[t]) < 2e-2, (t, "released, literal")
    assert rel(model.prefill(ids)[0], want[-1]) < 2e-2
    with pytest.raises(RuntimeError):
        model.layers[0].q_proj.state_dict()
    model.unprepack()
    assert all(m.qweight.numel() > 0 for layer in model.layers for m in layer.children())
    model._graph = None
    model.fuse_norm = True
    out, times, total = model.generate(ids[:4], 8, use_graph=True)
    out2, _, _ = model.generate(ids[:4], 8, use_graph=False)
    assert torch.equal(out, out2) and out.numel() == 8


@pytest.mark.parametrize("bits,prompt_len", [(4, 24), (3, 7)])
def test_batched_prefill_matches_token_steps(dec, bits, prompt_len):
    """The prompt in one batched pass (tiled GEMM kernel at 24 rows, small-batch kernel at 7): last
    position's logits against the dense reference and against feeding the prompt token by
    token; the KV caches agree with the step path's; decoding continues from the prefilled state."""
    print("[case] batched prefill", bits, prompt_len, flush=True)
    cfg = dec.DecoderConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                            num_key_value_heads=1, vocab_size=512, max_position_embeddings=48, w_bits=bits,
                            group_size=128, cherry_fraction=1 / 16)
    model = dec.CherryLlamaDecoder(cfg, seed=5)
    ids = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=torch.Generator().manual_seed(1))
    want = model.reference_logits(ids)[-1]
    stepped = model.step_logits(ids)[-1]
    k_step, v_step = model.k_cache.clone(), model.v_cache.clone()
    got = model.prefill(ids)[0]
    assert rel(got, want) < 2e-2 and rel(got, stepped) < 2e-2
    assert int(model.pos.item()) == prompt_len
    assert int(model.history[prompt_len - 1].item()) == int(got.argmax().item())
    assert rel(model.k_cache[:, :, :prompt_len], k_step[:, :, :prompt_len]) < 1e-2
    assert rel(model.v_cache[:, :, :prompt_len], v_step[:, :, :prompt_len]) < 1e-2
    assert not model.k_cache[:, :, prompt_len:].any()
    # the step that follows consumes the predicted token: teacher-forced reference on prompt + that token
    nxt = model.history[prompt_len - 1:prompt_len]
    model._step()
    want2 = model.reference_logits(torch.cat([ids.to(nxt.device), nxt]))[-1]
    assert rel(model.logits[0], want2) < 2e-2
    out, _, _ = model.generate(ids, 6, use_graph=True, batched_prefill=True)
    out2, _, _ = model.generate(ids, 6, use_graph=False, batched_prefill=True)
    assert out.numel() == 6 and torch.equal(out, out2) and int(out[0]) == int(nxt[0])


def test_saved_checkpoint_reloads_to_identical_logits(dec, tmp_path):
    """save_quantized -> from_quantized (reference file name and key names) gives a decoder whose
    token step reproduces the original's logits bit for bit."""
    print("[case] checkpoint round trip", flush=True)
    import utils as cq_utils
    cfg = dec.DecoderConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                            num_key_value_heads=1, vocab_size=512, max_position_embeddings=32, w_bits=4,
                            group_size=128, cherry_fraction=1 / 16)
    model = dec.CherryLlamaDecoder(cfg, seed=7)
    ids = torch.randint(0, cfg.vocab_size, (6,), generator=torch.Generator().manual_seed(0))
    want = model.step_logits(ids)
    cq_utils.save_quantized(model, str(tmp_path))
    loaded = cq_utils.from_quantized(str(tmp_path), prepack=False)
    assert loaded.layers[0].q_proj.qweight.is_cuda
    assert torch.equal(loaded.step_logits(ids), want)
    assert rel(want[-1], model.reference_logits(ids)[-1]) < 2e-2
    # the default: the recommended layers repacked on load (all seven linears of these small layers);
    # same weights, the stream kernels' rounding
    repacked = cq_utils.from_quantized(str(tmp_path))
    assert all(getattr(m, "_stream", None) is not None for m in repacked.layers[0].children())
    got = repacked.step_logits(ids)
    for t in range(ids.numel()):
        assert rel(got[t], want[t]) < 5e-3, t
    # a decode deployment: only the streams stay on the device; same logits as with both layouts
    lean = cq_utils.from_quantized(str(tmp_path), release_reference=True)
    assert all(m.qweight.numel() == 0 and m._stream is not None for m in lean.layers[1].children())
    assert torch.equal(lean.step_logits(ids), got)
    assert lean.step_bytes() == repacked.step_bytes()


def test_argmax_embed_tail_kernel(dec):
    """Greedy tail: argmax with the lowest index among equal maxima, history entry, embedding of
    the chosen token as next hidden state, position increment; odd vocabulary sizes included."""
    print("[case] argmax_embed", flush=True)
    lib = dec._lib
    torch.manual_seed(4)
    for vocab, hidden in ((32000, 4096), (517, 256), (8, 64)):
        embed = torch.randn(vocab, hidden, device="cuda").half()
        hid = torch.zeros(1, hidden, device="cuda").half()
        nxt = torch.full((1,), -1, dtype=torch.int64, device="cuda")
        hist = torch.full((16,), -1, dtype=torch.int64, device="cuda")
        pos = torch.tensor([3], dtype=torch.int32, device="cuda")
        for trial in range(4):
            logits = torch.randn(1, vocab, device="cuda").half()
            if trial == 1:  # a tie: the same maximum at two places
                logits[0, vocab - 1] = 9.0
                logits[0, vocab // 3] = 9.0
            if trial == 2:
                logits[0, 0] = 11.0
            lf = logits.float()[0]
            want = int((lf == lf.max()).nonzero()[0])  # lowest index among equal maxima
            p0 = int(pos)
            assert lib.cherryq_decode_argmax_embed_f16(logits.data_ptr(), vocab, embed.data_ptr(), hidden, hid.data_ptr(),
                                                       nxt.data_ptr(), hist.data_ptr(), hist.numel(), pos.data_ptr(),
                                                       stream()) == 0
            torch.cuda.synchronize()
            assert int(nxt) == want, (vocab, trial)
            assert int(pos) == p0 + 1 and int(hist[p0]) == want
            assert torch.equal(hid[0], embed[want])
    assert lib.cherryq_decode_argmax_embed_f16(None, 8, None, 8, None, None, None, 0, None, None) == -1


def _packed_host(m):
    return {b: getattr(m, b).cpu().numpy() for b in ("qweight", "scales", "cherry_weight", "cherry_indices")}


@pytest.mark.parametrize("bits", [4, 3])
@pytest.mark.parametrize("case", ["qkv_norm", "gate_up_norm", "down_silu_accumulate"])
def test_matvec_group_llama7b_shapes_against_the_c_oracle(dec, bits, case):
    """The grouped launch at the shapes and with the prologues the 7B decoder uses -- 3 x (4096 ->
    4096) behind a fused RMSNorm, 2 x (4096 -> 11008) behind a fused RMSNorm, 11008 -> 4096 on
    silu(gate) * up accumulating into the output -- against the C oracle's fused product of the
    prologue's result (rel-L2 1e-3), and bit for bit on activations whose prologue result is one-hot."""
    print("[case] matvec_group 7B shapes", bits, case, flush=True)
    from oracle import c_oracle
    import numpy as np
    K, widths = {"qkv_norm": (4096, (4096, 4096, 4096)), "gate_up_norm": (4096, (11008, 11008)),
                 "down_silu_accumulate": (11008, (4096,))}[case]
    gen = torch.Generator(device="cuda").manual_seed(17 + bits)
    cfg = dec.DecoderConfig(w_bits=bits, group_size=128, cherry_fraction=1 / 256)
    mods = [dec.random_packed_linear(cfg, K, n, gen, "cuda") for n in widths]
    packed = [_packed_host(m) for m in mods]
    f16 = lambda a: np.asarray(a).astype(np.float16)

    def run(vec, base=None, **kw):
        outs = [torch.full((1, n), 7.0, dtype=torch.float16, device="cuda") if base is None else
                torch.from_numpy(base[i]).cuda() for i, n in enumerate(widths)]
        for rep in range(2):  # the second call finds the workspace as the first one left it
            if rep and base is not None:
                for o, b in zip(outs, base):
                    o.copy_(torch.from_numpy(b))
            dec.matvec_group(mods, torch.from_numpy(vec).cuda(), outs, **kw)
        torch.cuda.synchronize()
        return [o.cpu().numpy() for o in outs]

    rng = np.random.default_rng(5)
    if case != "down_silu_accumulate":
        eps = 1e-6
        h = f16(rng.standard_normal((1, K)) * 3)
        nw = f16(rng.random(K) + 0.5)
        hf = h.astype(np.float64)
        act = f16(nw.astype(np.float64) * f16(hf / np.sqrt(np.mean(hf * hf) + eps)).astype(np.float64))
        got = run(h, norm_weight=torch.from_numpy(nw).cuda(), eps=eps)
        for o, p in zip(got, packed):
            assert rel(torch.from_numpy(o), torch.from_numpy(c_oracle.fused(act, p, bits, 128))) < 1e-3
        # one-hot through the norm: mean(x^2) + eps = 1 exactly for x = e_j and eps = 1 - 1/K, so the
        # normalised activation is norm_weight[j] * 1 (a power of two here): outputs are dense columns
        nw2 = f16(2.0 ** rng.integers(-2, 3, K))
        for j in (0, 1, 127, 128, 2049, K - 1, int(packed[0]["cherry_indices"][0]), int(packed[-1]["cherry_indices"][-1])):
            x = np.zeros((1, K), dtype=np.float16)
            x[0, j] = 1
            got = run(x, norm_weight=torch.from_numpy(nw2).cuda(), eps=1.0 - 1.0 / K)
            xa = np.zeros((1, K), dtype=np.float16)
            xa[0, j] = nw2[j]
            for o, p in zip(got, packed):
                with np.errstate(over="ignore"):
                    np.testing.assert_array_equal(o[0], f16(c_oracle.fused(xa, p, bits, 128)[0]), err_msg=f"column {j}")
    else:
        g = f16(rng.standard_normal((1, K)))
        u = f16(rng.standard_normal((1, K)))
        gf = g.astype(np.float64)
        act = f16(f16(gf / (1 + np.exp(-gf))).astype(np.float64) * u.astype(np.float64))
        base = [f16(rng.standard_normal((1, n))) for n in widths]
        got = run(u, base=base, vec_gate=torch.from_numpy(g).cuda(), accumulate=True)
        want = base[0].astype(np.float64) + c_oracle.fused(act, packed[0], bits, 128)
        assert rel(torch.from_numpy(got[0]), torch.from_numpy(want)) < 1e-3
        # silu(16) rounds to 16 in fp16, times up = 1/16: the staged activation is e_j exactly
        for j in (0, 1, 127, 128, 5000, K - 1, int(packed[0]["cherry_indices"][0]), int(packed[0]["cherry_indices"][-1])):
            g1 = f16(rng.standard_normal((1, K)))
            u1 = np.zeros((1, K), dtype=np.float16)
            g1[0, j], u1[0, j] = 16, 1 / 16
            x = np.zeros((1, K), dtype=np.float16)
            x[0, j] = 1
            got = run(u1, base=base, vec_gate=torch.from_numpy(g1).cuda(), accumulate=True)
            want = f16(base[0].astype(np.float64) + c_oracle.fused(x, packed[0], bits, 128))
            np.testing.assert_array_equal(got[0], want, err_msg=f"column {j}")


def test_positions_outside_the_cache_touch_nothing_and_poison_the_output(dec):
    """A position that is negative or at / beyond max_len must not index the KV cache: the rotary /
    cache-write kernels write nothing, the attention kernels read nothing and return NaN so that the
    mistake shows downstream."""
    print("[case] decode position guards", flush=True)
    lib = dec._lib
    nh, nkv, hd, ml = 4, 2, 128, 16
    torch.manual_seed(3)
    for bad in (ml, ml + 5, -1, -(2 ** 31)):
        kc = torch.randn(nkv, ml, hd, device="cuda").half()
        vc = torch.randn(nkv, ml, hd, device="cuda").half()
        kc0, vc0 = kc.clone(), vc.clone()
        q = torch.randn(1, nh * hd, device="cuda").half()
        k = torch.randn(1, nkv * hd, device="cuda").half()
        v = torch.randn(1, nkv * hd, device="cuda").half()
        pos = torch.tensor([bad], dtype=torch.int32, device="cuda")
        q1 = q.clone()
        assert lib.cherryq_decode_rope_cache_f16(q1.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                                 pos.data_ptr(), nh, nkv, hd, ml, 10000.0, stream()) == 0
        out = torch.zeros(1, nh * hd, device="cuda").half()
        assert lib.cherryq_decode_attention_f16(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(), pos.data_ptr(),
                                                nh, nkv, hd, ml, stream()) == 0
        out2 = torch.zeros(1, nh * hd, device="cuda").half()
        q2 = q.clone()
        assert lib.cherryq_decode_rope_attention_f16(q2.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(),
                                                     vc.data_ptr(), out2.data_ptr(), pos.data_ptr(), nh, nkv, hd, ml,
                                                     10000.0, stream()) == 0
        torch.cuda.synchronize()
        assert torch.equal(kc, kc0) and torch.equal(vc, vc0), bad
        assert torch.isnan(out).all() and torch.isnan(out2).all(), bad
    # the last valid position still works
    pos = torch.tensor([ml - 1], dtype=torch.int32, device="cuda")
    out = torch.zeros(1, nh * hd, device="cuda").half()
    assert lib.cherryq_decode_rope_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                                 out.data_ptr(), pos.data_ptr(), nh, nkv, hd, ml, 10000.0, stream()) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
