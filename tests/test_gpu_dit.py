"""GPU tests of the DiT block and the streaming generator on top of the NVFP4 kernels."""
import numpy as np
import pytest
import torch

import dit_oracle
import nvfp4_oracle as o
from helpers import bits_of, u8
from longlive_amd.dit import CausalDiT, DiTBlock, DiTConfig, StreamingGenerator
from longlive_amd.fouroversix import ModelQuantizationConfig, QuantizationConfig
from longlive_amd.utils import kv_cache as kvc
from longlive_amd.utils.quant import quantize_model_with_filter
from longlive_amd.utils.rope import build_rope_angles, rope_cos_sin

pytestmark = pytest.mark.gpu
KV = QuantizationConfig(scale_rule="mse")


def _f(t):
    return t.detach().float().cpu().numpy()


from helpers import block_oracle_params as _oracle_params  # noqa: E402


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


@pytest.mark.parametrize("dim,heads,ffn", [(256, 2, 512), (3072, 24, 14336)])
def test_block_against_oracle_with_cache(gpu, dim, heads, ffn):
    """Wan-shaped block, reduced (dim 256, 2 heads x 128, FFN 512) and at the full width of the benchmark model
    (dim 3072, 24 heads, FFN 14336); chunk = 2 frames x 64 tokens, two chunks so that the second one attends an
    FP4 slot.  Tolerance: relative Frobenius 6e-2 on the bf16
    block output: attention outputs that differ by ~1e-3 are re-quantized to FP4 three more times
    before the block output, which amplifies the difference (measured 3.4e-2); the stage-wise test
    below carries the tight bounds."""
    torch.manual_seed(0)
    F, h, w, T = 2, 8, 8, 16
    fs, L = h * w, 2 * 8 * 8
    block = DiTBlock(dim, ffn, heads).to(gpu)
    for m in block.modules():
        if isinstance(m, torch.nn.Linear):
            torch.nn.init.normal_(m.bias, std=0.1)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    params = _oracle_params(block)
    cache = kvc.initialize_kv_cache(1, L, 3, heads, 128, KV, gpu)[0]
    angles = build_rope_angles(128)
    g = torch.Generator().manual_seed(1)
    ctx = torch.randn(1, T, dim, generator=g).bfloat16()
    cached_k = cached_v = None
    for chunk in range(2):
        x = torch.randn(1, L, dim, generator=g).bfloat16()
        e0 = torch.randn(1, F, 6, dim, generator=g).bfloat16()
        cos, sin = rope_cos_sin(angles, F, h, w, start_frame=chunk * F, device=gpu)
        with torch.no_grad():
            y, (ce, le, info) = block(x.to(gpu), e0.to(gpu), cos, sin, ctx.to(gpu), cache, chunk * L, sink_tokens=L)
        ocs, osn = o.rope_cos_sin(F, h, w, start_frame=chunk * F)
        ref, rk, v = dit_oracle.block_forward(_f(x)[0], _f(e0)[0], _f(ctx)[0], params, ocs, osn, cached_k, cached_v,
                                              heads, fs)
        r = _rel(_f(y)[0], ref)
        print(f"block against oracle, dim {dim}, chunk {chunk}: relative Frobenius {r:.3e}")
        assert r <= 6e-2, (chunk, r)
        kvc.apply_cache_update(cache, ce, le, info, KV)
        # oracle cache: quantize-on-write of this chunk's un-smoothed K and V
        vals, sc, am, _ = o.quantize_to_fp4(o.f32_to_bf16(rk.reshape(-1, 128)), "mse")
        cached_k = o.kv_dequantize(vals, sc, am).reshape(L, heads, 128)
        vals, sc, am, _ = o.quantize_to_fp4(o.f32_to_bf16(v.reshape(-1, 128)), "mse")
        cached_v = o.kv_dequantize(vals, sc, am).reshape(L, heads, 128)


@pytest.mark.parametrize("dim,heads,ffn", [(256, 2, 512), (3072, 24, 14336)])
def test_block_stage_by_stage_against_oracle(gpu, dim, heads, ffn):
    """Every stage of the block forward on the GPU against the oracle's stage fed with the same
    (GPU-produced) input: elementwise stages bit-exact, W4A4 linears <= 1e-3 relative Frobenius,
    attention <= 2e-2 max-abs.  Once on a reduced block and once at the full width of the benchmark model
    (dim 3072, 24 heads, FFN 14336) on 128 tokens."""
    from longlive_amd import _native
    from longlive_amd.utils.adaln import adaln_modulate
    from longlive_amd.utils.quant import k_smooth
    from longlive_amd.utils.rope import rope_apply

    torch.manual_seed(0)
    F, h, w, T = 2, 8, 8, 16
    fs, L = h * w, 128
    block = DiTBlock(dim, ffn, heads).to(gpu)
    for m in block.modules():
        if isinstance(m, torch.nn.Linear):
            torch.nn.init.normal_(m.bias, std=0.1)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    p = _oracle_params(block)
    g = torch.Generator().manual_seed(1)
    ctx = torch.randn(1, T, dim, generator=g).bfloat16()
    x = torch.randn(1, L, dim, generator=g).bfloat16()
    e0 = torch.randn(1, F, 6, dim, generator=g).bfloat16()
    cos, sin = rope_cos_sin(build_rope_angles(128), F, h, w, 0, gpu)
    ocs, osn = o.rope_cos_sin(F, h, w, 0)

    def exact(name, got, ref):
        assert np.array_equal(_f(got).reshape(ref.shape), ref), name

    def one_ulp(name, got, ref):
        """Reductions over the channel dimension (layer norm, RMS norm) add 3072 terms in another order than
        numpy does: the fp32 statistics can differ in the last bit, which now and then moves a bf16 result to the
        neighbouring value.  Bit-exact at dim 256; at full width the bar of the adaLN parity test: <= 3.1e-2 (one
        bf16 ulp at the largest magnitudes here) on fewer than 5 in 1000."""
        g_, r_ = _f(got).reshape(ref.shape), ref
        if dim <= 256:
            assert np.array_equal(g_, r_), name
            return
        diff = np.abs(g_ - r_)
        assert diff.max() <= 3.1e-2 and (diff > 0).mean() < 5e-3, (name, diff.max(), (diff > 0).mean())

    def close(name, got, ref, tol=1e-3):
        assert _rel(_f(got).reshape(ref.shape), ref) <= tol, name

    def attn_close(name, got, ref):
        assert np.abs(_f(got).reshape(ref.shape) - ref).max() <= 2e-2, name

    fidx = np.arange(L) // fs
    with torch.no_grad():
        xg, eg, cg = x.to(gpu), e0.to(gpu), ctx.to(gpu)
        e = (block.modulation.unsqueeze(1) + eg).chunk(6, dim=2)
        eo = o.round_bf16(p["modulation"][None] + _f(e0)[0])
        exact("modulation", torch.cat(e, 2), eo)
        y = adaln_modulate(xg, e[1], e[0], fs)
        one_ulp("adaln1", y, o.adaln_modulate(_f(x)[0], eo[:, 1], eo[:, 0], fs))
        sa = block.self_attn
        ql = sa.q(y)
        close("q linear", ql, dit_oracle.linear_w4a4(_f(y)[0], p["self_attn.q.w"], p["self_attn.q.b"]))
        qn = sa.norm_q(ql)
        one_ulp("q rms", qn, o.rms_norm(_f(ql)[0], p["self_attn.norm_q"]))
        kn, vv = sa.norm_k(sa.k(y)), sa.v(y)
        rq = rope_apply(qn.view(L, heads, 128), cos, sin)
        exact("rope q", rq, o.rope_apply(_f(qn).reshape(L, heads, 128), ocs, osn))
        rk = rope_apply(kn.view(L, heads, 128), cos, sin)
        ks = k_smooth(rk.unsqueeze(0))[0]
        exact("k_smooth", ks, o.k_smooth(_f(rk)))
        a = _native.attention_bf16(rq, ks.contiguous(), vv.view(L, heads, 128).contiguous(), 128 ** -0.5)
        attn_close("self attention", a, o.attention(_f(rq), _f(ks), _f(vv).reshape(L, heads, 128)))
        ol = sa.o(a.reshape(1, L, dim))
        close("o linear", ol, dit_oracle.linear_w4a4(_f(a).reshape(L, dim), p["self_attn.o.w"], p["self_attn.o.b"]))
        x1 = xg + (ol.unflatten(1, (F, fs)) * e[2]).flatten(1, 2)
        exact("residual1", x1, o.round_bf16(_f(x)[0] + o.round_bf16(_f(ol)[0] * eo[fidx, 2])))
        n3 = block.norm3(x1)
        close("norm3", n3, dit_oracle.layer_norm_affine(_f(x1)[0], p["norm3.w"], p["norm3.b"]), 2e-3)
        ca = block.cross_attn
        cq, ck, cv = ca.norm_q(ca.q(n3)), ca.norm_k(ca.k(cg)), ca.v(cg)
        close("cross k", ck, o.rms_norm(dit_oracle.linear_w4a4(_f(ctx)[0], p["cross_attn.k.w"], p["cross_attn.k.b"]),
                                        p["cross_attn.norm_k"]), 2e-3)
        aa = _native.attention_bf16(cq.view(L, heads, 128), ck.view(T, heads, 128).contiguous(),
                                    cv.view(T, heads, 128).contiguous(), 128 ** -0.5)
        attn_close("cross attention", aa, o.attention(_f(cq).reshape(L, heads, 128), _f(ck).reshape(T, heads, 128),
                                                      _f(cv).reshape(T, heads, 128)))
        x2 = x1 + ca.o(aa.reshape(1, L, dim))
        y2 = adaln_modulate(x2, e[4], e[3], fs)
        h0 = block.ffn[0](y2)
        close("ffn.0", h0, dit_oracle.linear_w4a4(_f(y2)[0], p["ffn.0.w"], p["ffn.0.b"]))
        h1 = block.ffn[1](h0)
        close("gelu", h1, o.gelu_tanh(_f(h0)[0]), 2e-3)
        close("ffn.2", block.ffn[2](h1), dit_oracle.linear_w4a4(_f(h1)[0], p["ffn.2.w"], p["ffn.2.b"]))


def test_config4_full_size_block_runs_and_matches_a_dequantized_torch_graph(gpu):
    """Benchmark configuration 4 shape: dim 3072, 24 heads, FFN 14336, 2640 tokens, 512 text tokens, KV cache of
    4 full slots.  The CPU oracle is too slow at this size, so the check is against the same graph
    evaluated with torch on the GPU from the dequantized NVFP4 weights and fake-quantized activations
    (each of those conversions is verified bit-exactly elsewhere); tolerance 6e-2 relative Frobenius (see the first test)."""
    torch.manual_seed(3)
    dim, heads, ffn, F, h, w, T = 3072, 24, 14336, 3, 22, 40, 512
    fs, L = h * w, 3 * 22 * 40
    block = DiTBlock(dim, ffn, heads).to(gpu)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    cache = kvc.initialize_kv_cache(1, L, 5, heads, 128, KV, gpu)[0]
    g = torch.Generator().manual_seed(3)
    angles = build_rope_angles(128)
    ctx = torch.randn(1, T, dim, generator=g).bfloat16().to(gpu)
    for chunk in range(5):  # fill 4 slots, then measure the 5th chunk (sink + 3 window slots + itself)
        x = torch.randn(1, L, dim, generator=g).bfloat16().to(gpu)
        e0 = torch.randn(1, F, 6, dim, generator=g).bfloat16().to(gpu)
        cos, sin = rope_cos_sin(angles, F, h, w, start_frame=chunk * F, device=gpu)
        with torch.no_grad():
            y, (ce, le, info) = block(x, e0, cos, sin, ctx, cache, chunk * L, sink_tokens=L)
        if chunk < 4:
            kvc.apply_cache_update(cache, ce, le, info, KV)
    assert torch.isfinite(y.float()).all() and y.shape == (1, L, dim)

    from longlive_amd.fouroversix import quantize_to_fp4
    from longlive_amd.utils.quant import dequantize_kv_cache, k_smooth

    def lin(name, t):
        m = block.get_submodule(name)
        wd = m.quantized_weight().dequantize(torch.float32)
        td = quantize_to_fp4(t.reshape(-1, t.shape[-1])).dequantize(torch.float32)
        return ((td @ wd.T).bfloat16() + m.bias).reshape(*t.shape[:-1], -1)

    def rms(name, t):
        m = block.get_submodule(name)
        tf = t.float()
        return (tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16() * m.weight

    def rope(t):
        tc = torch.view_as_complex(t[0].double().reshape(L, heads, 64, 2))
        fr = torch.polar(torch.ones_like(cos.double()), torch.atan2(sin.double(), cos.double())).unsqueeze(1)
        return torch.view_as_real(tc * fr).flatten(2).bfloat16().unsqueeze(0)

    def attn(q_, k_, v_):
        return torch.nn.functional.scaled_dot_product_attention(
            q_.transpose(1, 2).float(), k_.transpose(1, 2).float(), v_.transpose(1, 2).float()).transpose(1, 2).bfloat16()

    with torch.no_grad():
        e = (block.modulation.unsqueeze(1) + e0).chunk(6, dim=2)
        ln = lambda t: torch.nn.functional.layer_norm(t.float(), (dim,), eps=1e-6).bfloat16()
        mod = lambda t, sc, sh: (ln(t).unflatten(1, (F, fs)) * (1 + sc) + sh).flatten(1, 2)
        y1 = mod(x, e[1], e[0])
        q_ = rope(rms("self_attn.norm_q", lin("self_attn.q", y1)).view(1, L, heads, 128))
        k_ = rope(rms("self_attn.norm_k", lin("self_attn.k", y1)).view(1, L, heads, 128))
        v_ = lin("self_attn.v", y1).view(1, L, heads, 128)
        ck = dequantize_kv_cache(cache["k"], 5, heads, L, torch.bfloat16, gpu)[:, :4 * L]
        cv = dequantize_kv_cache(cache["v"], 5, heads, L, torch.bfloat16, gpu)[:, :4 * L]
        a = attn(q_, torch.cat([ck, k_smooth(k_)], 1), torch.cat([cv, v_], 1))
        xr = x + (lin("self_attn.o", a.flatten(2)).unflatten(1, (F, fs)) * e[2]).flatten(1, 2)
        n3 = torch.nn.functional.layer_norm(xr.float(), (dim,), block.norm3.weight.float(), block.norm3.bias.float(), 1e-6).bfloat16()
        cq = rms("cross_attn.norm_q", lin("cross_attn.q", n3)).view(1, L, heads, 128)
        ckk = rms("cross_attn.norm_k", lin("cross_attn.k", ctx)).view(1, T, heads, 128)
        cvv = lin("cross_attn.v", ctx).view(1, T, heads, 128)
        xr = xr + lin("cross_attn.o", attn(cq, ckk, cvv).flatten(2))
        hdn = torch.nn.functional.gelu(lin("ffn.0", mod(xr, e[4], e[3])), approximate="tanh")
        xr = xr + (lin("ffn.2", hdn).unflatten(1, (F, fs)) * e[5]).flatten(1, 2)
    r = _rel(_f(y)[0], _f(xr)[0])
    assert r <= 6e-2, r


def test_streaming_generator_small_end_to_end(gpu):
    """Config-5-shaped run at reduced size: 2 layers, dim 256, 6 chunks of 2 frames (8x8 tokens), cache of
    3 blocks with a 1-block sink -> exercises fill, roll and the clean-context pass."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    gen = StreamingGenerator(cfg, gpu, seed=4)
    g = torch.Generator().manual_seed(4)
    noise = torch.randn(1, 12, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    out = gen.generate(noise, ctx)
    assert out.shape == noise.shape and torch.isfinite(out.float()).all()
    assert (out.float() - noise.float()).abs().max() > 1e-3
    c0 = gen.kv_cache[0]
    assert c0["_global_end"] == 12 * 64 and c0["_local_end"] == 3 * 128
    assert all(float(s.amax) > 0 for s in c0["k"])
    # determinism and cache reset
    gen2 = StreamingGenerator(cfg, gpu, seed=4)
    assert torch.equal(gen2.generate(noise, ctx), out)
    # the first chunk only depends on itself: generating just that chunk gives the same latents
    gen3 = StreamingGenerator(cfg, gpu, seed=4)
    assert torch.equal(gen3.generate(noise[:, :2], ctx), out[:, :2])


@pytest.mark.parametrize("clean", [False, True])
def test_streaming_generator_multi_shot_sink(gpu, clean):
    """Multi-shot mode at reduced size: global sink = first block, scene cuts at chunks 2 and 5 (with and without
    the clean recache).  The cache bookkeeping after the run has to equal the token-level policy oracle's, the
    frames before the first cut must not depend on the mode, and a second prompt takes effect from its chunk on."""
    import cache_policy_oracle as cpo

    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=8, sink_size=2)
    g = torch.Generator().manual_seed(6)
    noise = torch.randn(1, 16, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx_a, ctx_b = (torch.randn(10, 64, generator=g).bfloat16().to(gpu) for _ in range(2))
    contexts = [ctx_a] * 2 + [ctx_b] * 6
    cuts = (2, 5)
    gen = StreamingGenerator(cfg, gpu, seed=4, multi_shot_sink=True, shot_clean_recache=clean)
    out = gen.generate(noise, contexts, scene_cuts=cuts)
    assert torch.isfinite(out.float()).all()
    plain = StreamingGenerator(cfg, gpu, seed=4).generate(noise, contexts)
    assert torch.equal(out[:, :4], plain[:, :4])                  # nothing differs before the first roll / cut
    assert not torch.equal(out[:, 12:], plain[:, 12:])            # the protected prefix changes what later chunks see
    single = StreamingGenerator(cfg, gpu, seed=4).generate(noise, ctx_a)
    assert torch.equal(plain[:, :4], single[:, :4]) and not torch.equal(plain[:, 4:6], single[:, 4:6])

    blk, size = 2 * 64, 4 * 2 * 64
    st = cpo.new_state(size)
    for c in range(8):
        if c in cuts and clean:
            cpo.zero_kv_data(st, c * blk, blk)
        ids, upd = cpo.attend(st, c * blk, blk, blk, blk, size)
        cpo.apply(st, upd)
        if c in cuts:
            cpo.pin_current_chunk(st, blk, blk)
    for cache in gen.kv_cache:
        assert (cache["_global_end"], cache["_local_end"], cache["_pinned_start"], cache["_pinned_len"]) == \
            (st["global_end"], st["local_end"], st["pinned_start"], st["pinned_len"])
        assert int(cache["pinned_start"]) == st["pinned_start"] and int(cache["local_end_index"]) == st["local_end"]
    assert st["pinned_start"] == blk or clean                     # the pinned chunk ends up right behind the sink


def test_streaming_generator_multi_shot_rope_offset(gpu):
    """The temporal RoPE positions of every scene after a cut are shifted by scene index x offset: nothing changes
    before the first cut, the model's offset ends at (number of cuts) x offset, and a forward of the model with the
    offset equals a forward at the shifted frame position when the offset is a whole number of frames."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(9)
    noise = torch.randn(1, 10, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    gen = StreamingGenerator(cfg, gpu, seed=4, multi_shot_rope_offset=8.0)
    out = gen.generate(noise, ctx, scene_cuts=(2, 4))
    plain = StreamingGenerator(cfg, gpu, seed=4).generate(noise, ctx)
    assert torch.isfinite(out.float()).all()
    assert gen.model.rope_temporal_offset == 16.0
    assert torch.equal(out[:, :4], plain[:, :4]) and not torch.equal(out[:, 4:], plain[:, 4:])
    # one forward on an empty cache: offset 8 at frame 0 == no offset at frame 8 (tables agree to float32 rounding)
    m = gen.model
    x = noise[0, :2].transpose(0, 1).contiguous()
    t = torch.full((1, 2), 500.0, device=gpu)
    fs = 64
    def fresh():
        return kvc.initialize_kv_cache(cfg.num_layers, 2 * fs, 3, cfg.num_heads, 128, gen.kv_quant_config, gpu)
    m.rope_temporal_offset = 8.0
    a = m(x, t, ctx, fresh(), 0)
    m.rope_temporal_offset = 0.0
    cache = fresh()
    for c in cache:   # an empty cache whose stream position is frame 8
        c["_global_end"], c["_local_end"] = 8 * fs, 0
    b = m(x, t, ctx, cache, 8 * fs, apply_cache_updates=False)
    assert (a.float() - b.float()).abs().max() <= 0.02 * b.float().abs().max()


def test_streaming_generator_classifier_free_guidance(gpu):
    """guidance_scale != 1: every forward runs on the prompt and on the negative prompt with a cache each, the flow
    is uncond + s (cond - uncond).  With the negative prompt equal to the prompt the two forwards agree, so the
    result equals the unguided run up to the bf16 rounding of the combination; both caches end in the same state."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(10)
    noise = torch.randn(1, 8, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx, neg = (torch.randn(10, 64, generator=g).bfloat16().to(gpu) for _ in range(2))
    plain = StreamingGenerator(cfg, gpu, seed=4).generate(noise, ctx)
    gen = StreamingGenerator(cfg, gpu, seed=4, guidance_scale=3.0)
    with pytest.raises(ValueError):
        gen.generate(noise, ctx)
    same = gen.generate(noise, ctx, negative_context=ctx)
    assert (same.float() - plain.float()).abs().max() <= 0.05 * plain.float().abs().max()
    for a, b in zip(gen.kv_cache, gen.kv_cache_neg):
        assert a["_local_end"] == b["_local_end"] == 3 * 128 and a["_global_end"] == b["_global_end"] == 8 * 64
        assert torch.equal(a["k"][1].values, b["k"][1].values)
    gen.kv_cache = None
    guided = gen.generate(noise, ctx, negative_context=neg)
    assert torch.isfinite(guided.float()).all() and not torch.equal(guided, same)


def test_streaming_generator_continues_from_initial_latents(gpu):
    """Clean context frames fill the cache at timestep 0 exactly like the clean-context pass of a generated chunk,
    so continuing from the first chunk of a run reproduces the rest of that run bit for bit."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(11)
    noise = torch.randn(1, 10, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    full = StreamingGenerator(cfg, gpu, seed=4).generate(noise, ctx)
    gen = StreamingGenerator(cfg, gpu, seed=4)
    cont = gen.generate(noise[:, 4:], ctx, initial_latent=full[:, :4])
    assert cont.shape == full.shape and torch.equal(cont[:, :4], full[:, :4])
    assert torch.equal(cont[:, 4:], full[:, 4:])
    assert gen.kv_cache[0]["_global_end"] == 10 * 64
    with pytest.raises(NotImplementedError):
        gen.generate(noise[:, 4:], ctx, initial_latent=full[:, :3])


def test_streaming_generator_relative_rope(gpu):
    """While the window still starts at frame 0 of the stream, relative and absolute positions coincide, so the
    two modes may only differ by the bf16 rounding of cached-then-rotated keys."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(8)
    noise = torch.randn(1, 12, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    gen_rel, gen_abs = StreamingGenerator(cfg, gpu, seed=4, use_relative_rope=True), StreamingGenerator(cfg, gpu, seed=4)
    rel, ab = gen_rel.generate(noise, ctx), gen_abs.generate(noise, ctx)
    assert torch.isfinite(rel.float()).all()
    early = (rel[:, :6].float() - ab[:, :6].float()).abs().max().item()
    scale = ab.float().abs().max().item()
    assert early <= 0.06 * scale, (early, scale)
    assert gen_rel.kv_cache[0]["_local_end"] == gen_abs.kv_cache[0]["_local_end"] == 3 * 128


def test_packed_nvfp4_checkpoint_round_trip(gpu, tmp_path):
    """Export a quantized generator as a packed NVFP4 checkpoint, load it into a fresh bf16 model
    (utils/inference_utils.py:186-218 order: swap linears, drop master weights, strict load) and check
    that buffers and outputs are identical; a bf16 checkpoint of the same weights gives the same model."""
    from types import SimpleNamespace

    from longlive_amd.dit import CausalDiT
    from longlive_amd.utils import nvfp4_checkpoint as ck

    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    run_cfg = SimpleNamespace(model_quant_scale_rule="mse")
    gen = StreamingGenerator(cfg, gpu, seed=7)  # quantized (mse) and materialized
    path = tmp_path / "model_4o6.pt"
    saved = ck.save_nvfp4_checkpoint(path, gen.model, scale_rule="mse", model_name="tiny")
    assert saved["checkpoint_format"] == "longlive_generator_nvfp4" and saved["checkpoint_version"] == 1
    assert ck.is_nvfp4_state_dict(saved["generator"])
    assert not any(k.endswith("self_attn.q.weight") for k in saved["generator"])
    assert any(k.endswith("self_attn.q.quantized_weight_values") for k in saved["generator"])

    def fresh():
        torch.manual_seed(123)  # different init: everything must come from the checkpoint
        with torch.device(gpu):
            m = CausalDiT(cfg)
        m.rope_angles = m.rope_angles.cpu()
        return m

    loaded = ck.load_nvfp4_generator(fresh(), str(path), run_cfg).eval()
    a, b = gen.model.state_dict(), loaded.state_dict()
    assert a.keys() == b.keys()
    for k in a:
        assert torch.equal(a[k].cpu().view(torch.uint8) if a[k].dtype == torch.float8_e4m3fn else a[k].cpu(),
                           b[k].cpu().view(torch.uint8) if b[k].dtype == torch.float8_e4m3fn else b[k].cpu()), k

    g = torch.Generator().manual_seed(5)
    noise = torch.randn(1, 4, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    ref = gen.generate(noise, ctx)
    gen2 = StreamingGenerator(cfg, gpu, seed=99)
    gen2.model = loaded
    gen2.model.kv_quant_config = gen2.kv_quant_config
    assert torch.equal(gen2.generate(noise, ctx), ref)

    # TransformerEngine checkpoints and unknown versions are refused
    with pytest.raises(ValueError):
        ck.load_nvfp4_generator(fresh(), {"checkpoint_format": ck.TE_NVFP4_CHECKPOINT_FORMAT, "generator": {}})
    with pytest.raises(ValueError):
        ck.load_nvfp4_generator(fresh(), {**saved, "checkpoint_version": 2})
    # a checkpoint quantized under mse must not be loaded under the default static_6 configuration
    with pytest.raises(ValueError, match="scale rule"):
        ck.load_nvfp4_generator(fresh(), saved, SimpleNamespace())


def test_text_kv_cache_gives_identical_latents(gpu):
    """The per-prompt cache of the projected text K / V (crossattn_cache of the reference's interface) must not
    change a single bit of the output."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(8)
    noise = torch.randn(1, 6, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    a = StreamingGenerator(cfg, gpu, seed=4, cache_text_kv=True).generate(noise, ctx)
    b = StreamingGenerator(cfg, gpu, seed=4, cache_text_kv=False).generate(noise, ctx)
    assert torch.equal(a, b)
    # so must leaving out the cache writes of the denoising forwards, which the clean pass overwrites
    gen_c = StreamingGenerator(cfg, gpu, seed=4, skip_dead_cache_writes=False)
    c = gen_c.generate(noise, ctx)
    assert torch.equal(a, c)
    gen_a = StreamingGenerator(cfg, gpu, seed=4)
    gen_a.generate(noise, ctx)
    for la, lc in zip(gen_a.kv_cache, gen_c.kv_cache):
        assert la["_global_end"] == lc["_global_end"] and la["_local_end"] == lc["_local_end"]
        for sa, sc in zip(la["k"] + la["v"], lc["k"] + lc["v"]):
            assert torch.equal(sa.values, sc.values) and torch.equal(sa.amax, sc.amax)


def test_generator_with_the_unipc_sampler_follows_a_hand_stepped_scheduler(gpu):
    """sampler="unipc": every chunk is stepped by a fresh FlowUniPCMultistepScheduler exactly as the reference
    pipeline does (causal_diffusion_inference.py:566-612).  The first chunk is reproduced here by hand from the
    model's flow predictions, stepping the numpy oracle next to it."""
    import unipc_oracle as uo
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(9)
    noise = torch.randn(1, 4, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    gen = StreamingGenerator(cfg, gpu, seed=4, sampler="unipc", sample_shift=5.0)
    out = gen.generate(noise, ctx)
    assert out.shape == noise.shape and bool(torch.isfinite(out.float()).all())
    euler = StreamingGenerator(cfg, gpu, seed=4).generate(noise, ctx)
    assert not torch.equal(out, euler)

    ref = StreamingGenerator(cfg, gpu, seed=4, sampler="unipc", sample_shift=5.0)
    fs = (16 // cfg.patch_size[1]) * (16 // cfg.patch_size[2])
    ref.reset_cache(fs)
    sig, ts = uo.schedule(4, 5.0)
    x = noise[0, :2].transpose(0, 1).contiguous()
    ms, sig_hist, last, order, lower = [], [], None, 1, 0
    xo = x.double().cpu().numpy()
    with torch.no_grad():
        for i in range(4):
            tt = torch.full((1, 2), float(ts[i]), device=gpu)
            flow = ref.model(x, tt, ctx, ref.kv_cache, 0, apply_cache_updates=False).double().cpu().numpy()
            # the oracle in float64 on the model's own (bf16) trajectory
            m = x.double().cpu().numpy() - sig[i] * flow
            if i > 0:
                xo = uo.uni_c(last, ms, sig_hist, sig[i], m, order)
            else:
                xo = x.double().cpu().numpy()
            ms, sig_hist = (ms + [m])[-2:], (sig_hist + [sig[i]])[-2:]
            order = min(min(2, 4 - i), lower + 1)
            last = xo
            xo = uo.uni_p(xo, ms, sig_hist, sig[i + 1], order)
            lower = min(lower + 1, 2)
            x = torch.from_numpy(xo).to(gpu).bfloat16()
    # bf16 latents: the generator rounds after every step, the hand-stepped copy once per step as well
    diff = (out[0, :2].transpose(0, 1).float() - x.float()).abs().max().item()
    assert diff <= 2 * 2.0 ** -7 * out.float().abs().max().item(), diff  # two bf16 ulps of the largest latent


@pytest.mark.parametrize("time_gain,disp_tol,latent_tol", [(1.0, 4e-2, 1.5e-2), (40.0, 1e-1, 6e-2)])
def test_streaming_generator_against_the_chunk_loop_oracle(gpu, time_gain, disp_tol, latent_tol):
    """The generator on the GPU against the CPU restatement of the reference's chunk loop (oracle/generator_oracle.py:
    model forward around the blocks, four Euler / flow steps at 1000/750/500/250, timestep-0 recache, cache fill and
    roll), latent by latent.  2 layers, dim 256, 6 chunks of 2 frames (128 tokens), cache of 3 blocks with a 1-block
    sink, so chunks 3-5 each roll the window.

    Tolerance, per chunk: relative Frobenius error of the displacement (latent - noise, the integral of the
    predicted flow) <= 4e-2 and of the latent itself <= 1.5e-2 (measured 1.5e-2 and 4.5e-3: the FP4
    re-quantization of activations that differ in the last bf16 bit flips a few codes per forward).
    With the random initialisation the model barely reacts to the timestep, so a second case multiplies the first
    time-embedding weight by 40: the modulation then dominates, the errors grow with it (tolerance 1e-1 / 6e-2,
    measured 6.4e-2 / 3.8e-2), and leaving the timestep-0 pass out of the oracle moves every later chunk by more
    than 2e-1 (measured 2.7e-1 to 3.3e-1) -- the control that the comparison sees that pass."""
    import generator_oracle as go
    from helpers import generator_oracle_params
    from longlive_amd.utils.quant import dequantize_kv_cache

    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    gen = StreamingGenerator(cfg, gpu, seed=4)
    with torch.no_grad():
        gen.model.time_embedding[0].weight.mul_(time_gain)
    g = torch.Generator().manual_seed(4)
    noise = torch.randn(1, 12, 8, 16, 16, generator=g).bfloat16()
    ctx = torch.randn(10, 64, generator=g).bfloat16()
    out = gen.generate(noise.to(gpu), ctx.to(gpu)).cpu()
    P = generator_oracle_params(gen.model)
    ref, caches = go.generate(P, cfg, noise, ctx)

    def err(a, b, c):
        sl = slice(2 * c, 2 * c + 2)
        a, b, n = _f(a[0, sl]), _f(b[0, sl]), _f(noise[0, sl])
        return _rel(a - n, b - n), _rel(a, b)

    for c in range(6):
        d_err, l_err = err(out, ref, c)
        assert d_err <= disp_tol and l_err <= latent_tol, (c, d_err, l_err)
    if time_gain > 1:
        control, _ = go.generate(P, cfg, noise, ctx, recache=False)
        for c in range(1, 6):
            assert err(control, ref, c)[0] > 2e-1, c
    # cache state: same bookkeeping, and the slots hold what the oracle's cache holds: slot amax within 3 % (10 % in the amplified case), content
    # within 0.2 relative Frobenius (two FP4 quantizations of inputs that differ in the last bf16 bits differ by
    # whole e2m1 steps where a value sits next to a rounding boundary or the block's 4-or-6 choice flips; the
    # quantization noise of NVFP4 itself is about 0.1)
    blk = 128
    for layer, (cache, oc) in enumerate(zip(gen.kv_cache, caches)):
        st = oc["policy"]
        assert (cache["_global_end"], cache["_local_end"]) == (st["global_end"], st["local_end"]) == (12 * 64, 3 * blk)
        for name in ("k", "v"):
            got = _f(dequantize_kv_cache(cache[name], 3, 2, blk, torch.bfloat16, gpu)[0])
            for slot in range(3):
                chunk = int(st["buf"][slot * blk]) // blk
                assert _rel(got[slot * blk:(slot + 1) * blk], oc[name][chunk]) <= 0.2, (layer, name, slot)
                assert abs(float(cache[name][slot].amax) / oc[name + "_amax"][chunk] - 1) <= max(0.03, disp_tol), (layer, name, slot)
        assert [int(st["buf"][s * blk]) // blk for s in range(3)] == [0, 4, 5]


def test_config5_full_size_generator_fills_and_rolls_the_window(gpu, monkeypatch):
    """Benchmark configuration 5 at full size (30 blocks, dim 3072, 24 heads, FFN 14336, chunks of 3 latent frames
    = 2640 tokens, FP4 cache of 5 blocks = sink 3 + window 12 frames, timesteps 1000/750/500/250 + the timestep-0
    recache pass), run for 6 chunks: five fill the cache, the sixth rolls it.  The CPU oracle of the whole loop is
    out of reach at this size (184 TFLOP per chunk), so the checks are: finite, non-trivial latents; per-layer cache
    bookkeeping equal to the token-level policy oracle's; every slot of layer 0 holding, bit for bit, the bytes
    written for the chunk the policy oracle places there; and the newest slot's bytes equal to the CPU oracle's
    quantization of the rotated K (and of V) the model produced for that chunk in its recache pass."""
    import cache_policy_oracle as cpo
    from longlive_amd.dit import model as dit_model

    cfg = DiTConfig()
    gen = StreamingGenerator(cfg, gpu, seed=4)
    g = torch.Generator().manual_seed(4)
    n_chunks, fs, blk = 6, 880, 2640
    noise = torch.randn(1, 3 * n_chunks, 48, 44, 80, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(512, 4096, generator=g).bfloat16().to(gpu)

    written = {}          # chunk -> (K bytes, V bytes, K amax) of layer 0 right after the chunk's recache pass
    produced = {}         # chunk -> (rotated K, V) bf16 handed to the cache update of layer 0
    real_update = kvc.apply_cache_update

    def recording_update(cache, current_end, local_end_index, info, kv_cfg):
        real_update(cache, current_end, local_end_index, info, kv_cfg)
        if cache is gen.kv_cache[0] and info is not None:
            chunk = current_end // blk - 1
            slot = info["local_start_index"] // blk
            written[chunk] = (cache["k"][slot].values.clone(), cache["v"][slot].values.clone(),
                              cache["k"][slot].scale_factors.clone(), float(cache["k"][slot].amax))
            produced[chunk] = (info["new_k"], info["new_v"])

    monkeypatch.setattr(dit_model.kvc, "apply_cache_update", recording_update)
    out = gen.generate(noise, ctx)
    assert out.shape == noise.shape and torch.isfinite(out.float()).all()
    moved = (out.float() - noise.float()).norm() / noise.float().norm()
    assert 0.01 < float(moved) < 10.0
    assert sorted(written) == list(range(n_chunks))

    # policy oracle: five forwards per chunk, each applying its update, as the reference does
    st = cpo.new_state(5 * blk)
    for c in range(n_chunks):
        for _ in range(5):
            ids, upd = cpo.attend(st, c * blk, blk, cfg.sink_size * fs, 0, cfg.local_attn_size * fs)
            cpo.apply(st, upd)
    holds = [int(st["buf"][s * blk]) // blk for s in range(5)]
    assert holds == [0, 2, 3, 4, 5]
    for cache in gen.kv_cache:
        assert (cache["_global_end"], cache["_local_end"]) == (st["global_end"], st["local_end"])
        assert int(cache["global_end_index"]) == st["global_end"] and int(cache["local_end_index"]) == st["local_end"]
    c0 = gen.kv_cache[0]
    for slot, chunk in enumerate(holds):
        kb, vb, ksb, kam = written[chunk]
        assert torch.equal(c0["k"][slot].values, kb) and torch.equal(c0["v"][slot].values, vb), (slot, chunk)
        assert torch.equal(c0["k"][slot].scale_factors.view(torch.uint8), ksb.view(torch.uint8))
        assert float(c0["k"][slot].amax) == kam == float(produced[chunk][0].float().abs().max())
    # newest slot against the CPU oracle's quantization of what the model produced
    for name, t in zip(("k", "v"), produced[n_chunks - 1]):
        vals, sc, am, _ = o.quantize_to_fp4(bits_of(t[0].reshape(-1, 128)), "mse")
        slot = c0[name][4]
        assert float(slot.amax) == float(am)
        assert np.array_equal(u8(slot.scale_factors), sc) and np.array_equal(u8(slot.values), vals), name


@pytest.mark.parametrize("clean", [False, True])
def test_skipping_dead_cache_writes_is_invisible_in_multi_shot_mode(gpu, clean):
    """Leaving out the cache writes of the denoising forwards (which the timestep-0 pass overwrites) must not
    change a bit of the latents or of the final cache in multi-shot mode either: global sink, scene cuts at
    chunks 2 and 5 (pinned chunks that float to the front while the window rolls), with and without the clean
    recache."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=8, sink_size=2)
    g = torch.Generator().manual_seed(12)
    noise = torch.randn(1, 16, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    gens = [StreamingGenerator(cfg, gpu, seed=4, multi_shot_sink=True, shot_clean_recache=clean,
                               skip_dead_cache_writes=skip) for skip in (True, False)]
    a, b = (gen.generate(noise, ctx, scene_cuts=(2, 5)) for gen in gens)
    assert torch.equal(a, b)
    for la, lb in zip(gens[0].kv_cache, gens[1].kv_cache):
        for key in ("_global_end", "_local_end", "_pinned_start", "_pinned_len"):
            assert la[key] == lb[key], key
        for sa, sb in zip(la["k"] + la["v"], lb["k"] + lb["v"]):
            assert torch.equal(sa.values, sb.values) and torch.equal(sa.amax, sb.amax)


def test_head_modulation_through_the_adaln_kernel_matches_the_eager_graph(gpu):
    """CausalHead (wan_5b/modules/causal_model.py:933-959): norm(x) * (1 + e[1]) + e[0] runs through the adaLN
    kernel; against the same expression evaluated by torch's bf16 operations (each intermediate rounded to bf16) the
    head output may differ by the last bit of the modulated activations only."""
    from longlive_amd.dit.model import CausalHead

    torch.manual_seed(5)
    dim, F, fs = 512, 3, 40
    head = CausalHead(dim, 8, (1, 2, 2)).to(gpu).to(torch.bfloat16)
    torch.nn.init.normal_(head.head.weight, std=0.05)
    g = torch.Generator().manual_seed(6)
    x = (torch.randn(1, F * fs, dim, generator=g) * 3).bfloat16().to(gpu)
    e = torch.randn(1, F, 1, dim, generator=g).bfloat16().to(gpu)
    with torch.no_grad():
        got = head(x, e)
        em = (head.modulation.unsqueeze(1) + e).chunk(2, dim=2)
        ln = torch.nn.functional.layer_norm(x.float(), (dim,), eps=head.norm.eps).bfloat16()
        ref = head.head(ln.unflatten(1, (F, fs)) * (1 + em[1]) + em[0])
    assert got.shape == ref.shape == (1, F, fs, 32)
    assert (got.float() - ref.float()).abs().max() <= 2.0 ** -6 * ref.float().abs().max()


def test_modulation_of_all_blocks_in_one_operation_is_what_each_block_would_form(gpu):
    """The model adds its blocks' modulation parameters to the time projection in one operation per forward; each
    slice is bit for bit the block's own ``modulation.unsqueeze(1) + e``, follows a parameter that is written in
    place, and the generated latents are those of the block-by-block path."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=3, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    gen = StreamingGenerator(cfg, gpu, seed=9)
    model = gen.model
    g = torch.Generator().manual_seed(9)
    e0 = torch.randn(1, 2, 6, 256, generator=g).to(gpu).to(model.blocks[0].modulation.dtype)
    with torch.no_grad():
        for _ in range(2):
            stacked = model._stacked_modulation().unsqueeze(2) + e0.unsqueeze(0)
            for i, b in enumerate(model.blocks):
                assert torch.equal(stacked[i], b.modulation.unsqueeze(1) + e0)
            model.blocks[1].modulation.mul_(2.0)          # an in-place write must not leave a stale stack behind
    noise = torch.randn(1, 4, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    out = gen.generate(noise, ctx)
    gen2 = StreamingGenerator(cfg, gpu, seed=9)
    with torch.no_grad():
        gen2.model.blocks[1].modulation.mul_(4.0)
    block_forward = DiTBlock.forward
    def per_block(self, *args, modulated=None, **kwargs):   # the path without the stacked tensor
        return block_forward(self, *args, modulated=None, **kwargs)
    DiTBlock.forward = per_block
    try:
        ref = gen2.generate(noise, ctx)
    finally:
        DiTBlock.forward = block_forward
    assert torch.equal(out, ref)


def test_block_forward_recorded_into_a_graph_replays_bit_for_bit(gpu):
    """One DiT block forward over an FP4 cache slot recorded into a HIP graph (some twenty kernels of the library,
    among them the one-launch normalize-and-quantize kernels, whose workgroups meet through the sink) and replayed
    with new inputs.  A recorded launch runs again with the epoch it was recorded with, so the tickets of the recording come from a ReplayableAmaxSink, whose first recorded launch moves every epoch of
    the replay past those of the previous one.  Each of four replays - with eager forwards of the same block,
    which use the device's own sink, and synchronisations in between - must equal the eager result bit for bit;
    a replay that met stale maxima of an earlier replay would quantize against too large an amax."""
    from longlive_amd import _native

    torch.manual_seed(0)
    dim, heads, ffn, F, h, w, T = 256, 2, 512, 2, 8, 8, 16
    L = F * h * w
    block = DiTBlock(dim, ffn, heads).to(gpu)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    cache = kvc.initialize_kv_cache(1, L, 3, heads, 128, KV, gpu)[0]
    cos0, sin0 = rope_cos_sin(build_rope_angles(128), F, h, w, 0, gpu)
    cos1, sin1 = rope_cos_sin(build_rope_angles(128), F, h, w, F, gpu)
    g = torch.Generator().manual_seed(3)

    def inputs(scale):
        return ((torch.randn(1, L, dim, generator=g) * scale).bfloat16().to(gpu),
                torch.randn(1, F, 6, dim, generator=g).bfloat16().to(gpu),
                torch.randn(1, T, dim, generator=g).bfloat16().to(gpu))

    with torch.no_grad():
        x, e0, ctx = inputs(1.0)  # chunk 0 fills slot 0
        _, (ce, le, info) = block(x, e0, cos0, sin0, ctx, cache, 0, sink_tokens=L)
        kvc.apply_cache_update(cache, ce, le, info, KV)
        cases = [inputs(s) for s in (8.0, 1.0, 0.05, 3.0)]  # amax falls and rises between replays
        eager = [block(x, e0, cos1, sin1, ctx, cache, L, sink_tokens=L)[0].clone() for x, e0, ctx in cases]

        static = [t.clone() for t in cases[0]]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), _native.attention_policy("narrow"):  # no allocation inside the recording
            block(*static[:2], cos1, sin1, static[2], cache, L, sink_tokens=L)
        torch.cuda.current_stream().wait_stream(side)
        sink = _native.ReplayableAmaxSink(gpu)
        graph = torch.cuda.CUDAGraph()
        with _native.attention_policy("narrow"), torch.cuda.graph(graph, stream=side), sink:
            y_static = block(*static[:2], cos1, sin1, static[2], cache, L, sink_tokens=L)[0]
        assert sink.entry[1] >= 5  # the recording used the graph's sink
        for i, case in enumerate(cases):
            for dst, src in zip(static, case):
                dst.copy_(src)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_static, eager[i]), i
            other = block(*cases[(i + 1) % 4][:2], cos1, sin1, cases[(i + 1) % 4][2], cache, L, sink_tokens=L)[0]
            assert torch.equal(other, eager[(i + 1) % 4])
            torch.cuda.synchronize()


def test_cache_write_takes_the_k_and_v_maxima_from_their_producers(gpu):
    """The chunk's roped K and its V are quantized into the cache after the forward.  Their producers (the norm +
    RoPE kernel, the V projection's epilogue) leave the tensor maxima in the layer's own amax sinks, and the cache
    write reads them instead of reducing the tensors again: the slot bytes and the slot amax equal those of a write
    that computes the maxima itself, and a second forward's tickets replace the first's."""
    from longlive_amd import _native

    torch.manual_seed(0)
    dim, heads, ffn, F, h, w, T = 256, 2, 512, 2, 8, 8, 16
    L = F * h * w
    block = DiTBlock(dim, ffn, heads).to(gpu)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    cos, sin = rope_cos_sin(build_rope_angles(128), F, h, w, 0, gpu)
    g = torch.Generator().manual_seed(4)
    cache = kvc.initialize_kv_cache(1, L, 2, heads, 128, KV, gpu)[0]
    plain = kvc.initialize_kv_cache(1, L, 2, heads, 128, KV, gpu)[0]
    with torch.no_grad():
        for scale in (4.0, 0.25):  # the second forward writes the same slot again, with smaller maxima
            x = (torch.randn(1, L, dim, generator=g) * scale).bfloat16().to(gpu)
            e0 = torch.randn(1, F, 6, dim, generator=g).bfloat16().to(gpu)
            ctx = torch.randn(1, T, dim, generator=g).bfloat16().to(gpu)
            _, (ce, le, info) = block(x, e0, cos, sin, ctx, cache, 0, sink_tokens=L)
            assert isinstance(info["new_k_amax"], _native.AmaxTicket) and isinstance(info["new_v_amax"], _native.AmaxTicket)
            assert info["new_k_amax"].parts is not info["new_v_amax"].parts
            without = {k: v for k, v in info.items() if not k.endswith("_amax")}
            kvc.apply_cache_update(plain, ce, le, without, KV)
            kvc.apply_cache_update(cache, ce, le, info, KV)
            for name, new in (("k", info["new_k"]), ("v", info["new_v"])):
                a, b = cache[name][0], plain[name][0]
                assert float(a.amax) == float(b.amax) == float(new.float().abs().max())
                assert torch.equal(a.values, b.values) and np.array_equal(u8(a.scale_factors), u8(b.scale_factors))
            cache["_global_end"] = cache["_local_end"] = plain["_global_end"] = plain["_local_end"] = 0  # write slot 0 again


def test_streaming_decode_hook_decodes_every_chunk_in_order_on_a_side_stream(gpu):
    """Streaming decode (pipeline/causal_diffusion_inference.py:443-456, 666-683): each finished chunk goes to a
    decoder on a side stream while the generator carries on.  The decoder here keeps state between chunks like
    the reference's cached VAE decode (a running sum of everything seen so far enters each output), so a chunk
    decoded out of order, twice, or before its latents are final would show.  The decoded chunks must equal the
    same decoder run over the finished latents afterwards, and the latents those of a run without the hook."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)

    def build():
        return StreamingGenerator(cfg, gpu, seed=11)

    gen = build()
    g = torch.Generator().manual_seed(12)
    noise = torch.randn(1, 10, 8, 16, 16, generator=g).bfloat16().to(gpu)
    context = torch.randn(6, 64, generator=g).bfloat16().to(gpu)
    plain = gen.generate(noise, context)

    class Decoder:
        def __init__(self):
            self.seen = torch.zeros((), device=gpu, dtype=torch.float32)
            self.calls = 0

        def __call__(self, latents):
            assert latents.shape[0] == 1 and latents.shape[1] == gen.cfg.in_dim
            self.calls += 1
            self.seen = self.seen + latents.float().sum()
            up = torch.nn.functional.interpolate(latents[0].float(), scale_factor=2.0, mode="nearest")
            return (up + self.seen).clamp_(-50, 50)

    gen2 = build()
    streamed = Decoder()
    latents, chunks = gen2.generate(noise, context, decode_chunk=streamed)
    torch.cuda.synchronize()
    assert torch.equal(latents, plain)
    nb = gen.cfg.num_frame_per_block
    assert streamed.calls == len(chunks) == noise.shape[1] // nb
    offline = Decoder()
    for i, chunk in enumerate(chunks):
        want = offline(plain[:, i * nb:(i + 1) * nb].transpose(1, 2).contiguous())
        assert torch.equal(chunk, want), i


def test_time_conditioning_cached_per_timestep_value_gives_identical_latents(gpu):
    """The time embedding, its projection and modulation + e0 are computed once per timestep value when the caller
    names the value (the streaming generator does: five values per run); the latents are bit for bit those of a run
    that recomputes them in every forward, and a parameter written in place invalidates what was kept."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=6, sink_size=2)
    g = torch.Generator().manual_seed(12)
    noise = torch.randn(1, 6, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    gen = StreamingGenerator(cfg, gpu, seed=12)
    out = gen.generate(noise, ctx)
    kept = [k for k in gen.model._time_cache if k != "version"]
    assert len(kept) == 5 and {k[0][0] for k in kept} == {1000.0, 750.0, 500.0, 250.0, 0.0}
    gen2 = StreamingGenerator(cfg, gpu, seed=12)
    forward = type(gen2.model).forward

    def uncached(self, *args, timestep_key=None, **kwargs):
        return forward(self, *args, timestep_key=None, **kwargs)
    type(gen2.model).forward = uncached
    try:
        ref = gen2.generate(noise, ctx)
    finally:
        type(gen2.model).forward = forward
    assert torch.equal(out, ref)
    with torch.no_grad():
        gen.model.time_projection[1].bias.add_(0.5)
        gen2.model.time_projection[1].bias.add_(0.5)
    gen.kv_cache = gen2.kv_cache = None
    again = gen.generate(noise, ctx)
    type(gen2.model).forward = uncached
    try:
        ref2 = gen2.generate(noise, ctx)
    finally:
        type(gen2.model).forward = forward
    assert torch.equal(again, ref2) and not torch.equal(again, out)


@pytest.mark.parametrize("dim,heads,ffn,F,h,w", [(256, 2, 512, 2, 8, 8), (3072, 24, 14336, 3, 22, 40)])
def test_normalizing_and_quantizing_in_one_launch_leaves_the_block_bit_identical(gpu, dim, heads, ffn, F, h, w):
    """The three normalizations of a block that feed quantized layers (adaLN ahead of self-attention and of the
    FFN, norm3 ahead of cross-attention) produce the layers' NVFP4 operand directly; the block's output and the
    K / V it hands to the cache are those of the separate operations, bit for bit."""
    torch.manual_seed(1)
    L, T = F * h * w, 32
    block = DiTBlock(dim, ffn, heads).to(gpu).bfloat16()
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    cache = kvc.initialize_kv_cache(1, L, 3, heads, 128, KV, gpu)[0]
    cos, sin = rope_cos_sin(build_rope_angles(128), F, h, w, 0, gpu)
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(1, L, dim, generator=g) * 2).bfloat16().to(gpu)
    e = torch.randn(1, F, 6, dim, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(1, T, dim, generator=g).bfloat16().to(gpu)
    outs = []
    with torch.no_grad():
        for fuse in (True, False):
            block.fuse_norm_quantize = fuse
            y, (_, _, info) = block(x, e, cos, sin, ctx, cache, 0, sink_tokens=L)
            outs.append((y.clone(), info["new_k"].clone(), info["new_v"].clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("relative", [False, True])
def test_leaving_out_the_unread_tail_of_the_clean_context_pass_changes_nothing(gpu, relative):
    """The clean-context pass of a chunk (timestep 0, pipeline/causal_diffusion_inference.py:639-647) is run for its
    cache writes; its prediction has no reader.  With the last block stopped behind its K / V producers and the head
    left out, the latents and every byte of the cache are those of the full pass - for the plain run, with scene
    cuts, a continuation from given latents, and relative RoPE (whose cache holds un-rotated keys)."""
    cfg = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=8, out_dim=8, text_dim=64, text_len=16,
                    num_frame_per_block=2, local_attn_size=8, sink_size=2)
    g = torch.Generator().manual_seed(13)
    noise = torch.randn(1, 12, 8, 16, 16, generator=g).bfloat16().to(gpu)
    first = torch.randn(1, 2, 8, 16, 16, generator=g).bfloat16().to(gpu)
    ctx = torch.randn(10, 64, generator=g).bfloat16().to(gpu)
    gens = [StreamingGenerator(cfg, gpu, seed=4, multi_shot_sink=not relative, use_relative_rope=relative,
                               skip_dead_recache_tail=skip) for skip in (True, False)]
    cuts = () if relative else (2, 4)
    a, b = (gen.generate(noise, ctx, scene_cuts=cuts, initial_latent=first) for gen in gens)
    assert torch.equal(a, b)
    for la, lb in zip(gens[0].kv_cache, gens[1].kv_cache):
        for key in ("_global_end", "_local_end", "_pinned_start", "_pinned_len"):
            assert la[key] == lb[key], key
        for sa, sb in zip(la["k"] + la["v"], lb["k"] + lb["v"]):
            assert torch.equal(sa.values, sb.values) and torch.equal(sa.amax, sb.amax)
            assert torch.equal(sa.scale_factors.view(torch.uint8), sb.scale_factors.view(torch.uint8))
