"""CPU pins of the chunk-loop oracle (oracle/generator_oracle.py): closed forms and invariants that a wrong sigma,
a missing timestep-0 pass, a wrong roll or a transposed patch layout would fail."""
import numpy as np
import pytest
import torch

import generator_oracle as go
import nvfp4_oracle as o
from longlive_amd.dit import DiTConfig

CFG = DiTConfig(dim=256, ffn_dim=512, num_heads=2, num_layers=2, in_dim=4, out_dim=4, text_dim=32, text_len=8,
                num_frame_per_block=1, local_attn_size=3, sink_size=1)
H = W = 8          # latent size: 4 x 4 patches = 16 tokens per frame


def _qweight(rng, n, k, scale=0.05):
    w = o.round_bf16((rng.standard_normal((n, k)) * scale).astype(np.float32))
    v, s, a, pad = o.quantize_to_fp4(o.f32_to_bf16(w), "mse")
    return dict(values=v, scales=s, amax=a, rule="mse", padded=pad, orig=w.shape)


def make_params(cfg, seed=0, head_weight_scale=0.05, head_bias=None):
    rng = np.random.default_rng(seed)
    t = lambda *shape, s=0.05: torch.from_numpy((rng.standard_normal(shape) * s).astype(np.float32)).bfloat16()
    pd = cfg.in_dim * int(np.prod(cfg.patch_size))
    P = {"patch_embedding.weight": t(cfg.dim, pd, s=0.2), "patch_embedding.bias": t(cfg.dim),
         "time_embedding.0.weight": t(cfg.dim, cfg.freq_dim), "time_embedding.0.bias": t(cfg.dim),
         "time_embedding.2.weight": t(cfg.dim, cfg.dim), "time_embedding.2.bias": t(cfg.dim),
         "time_projection.1.weight": t(6 * cfg.dim, cfg.dim), "time_projection.1.bias": t(6 * cfg.dim, s=0.3),
         "text_embedding.0.weight": t(cfg.dim, cfg.text_dim), "text_embedding.0.bias": t(cfg.dim),
         "text_embedding.2.weight": t(cfg.dim, cfg.dim), "text_embedding.2.bias": t(cfg.dim),
         "head.modulation": t(1, 2, cfg.dim),
         "head.head.weight": t(cfg.out_dim * int(np.prod(cfg.patch_size)), cfg.dim, s=head_weight_scale),
         "head.head.bias": (t(cfg.out_dim * int(np.prod(cfg.patch_size))) if head_bias is None else
                            torch.full((cfg.out_dim * int(np.prod(cfg.patch_size)),), head_bias).bfloat16()),
         "blocks": []}
    for _ in range(cfg.num_layers):
        b = {"modulation": o.round_bf16((rng.standard_normal((6, cfg.dim)) / 16).astype(np.float32))}
        for name in ("self_attn.q", "self_attn.k", "self_attn.v", "self_attn.o", "cross_attn.q", "cross_attn.k",
                     "cross_attn.v", "cross_attn.o"):
            b[name + ".w"] = _qweight(rng, cfg.dim, cfg.dim)
            b[name + ".b"] = o.round_bf16((rng.standard_normal(cfg.dim) * 0.02).astype(np.float32))
        b["ffn.0.w"], b["ffn.0.b"] = _qweight(rng, cfg.ffn_dim, cfg.dim), np.zeros(cfg.ffn_dim, np.float32)
        b["ffn.2.w"], b["ffn.2.b"] = _qweight(rng, cfg.dim, cfg.ffn_dim), np.zeros(cfg.dim, np.float32)
        for name in ("self_attn.norm_q", "self_attn.norm_k", "cross_attn.norm_q", "cross_attn.norm_k"):
            b[name] = np.ones(cfg.dim, np.float32)
        b["norm3.w"], b["norm3.b"] = np.ones(cfg.dim, np.float32), np.zeros(cfg.dim, np.float32)
        P["blocks"].append(b)
    return P


def _inputs(frames, seed=1, grid=False):
    g = torch.Generator().manual_seed(seed)
    noise = torch.randn(1, frames, CFG.in_dim, H, W, generator=g)
    if grid:   # multiples of 1/16 within [-4, 4]: every Euler step of the closed-form test is exact in bf16
        noise = (noise.clamp(-4, 4) * 16).round() / 16
    return noise.bfloat16(), torch.randn(5, CFG.text_dim, generator=g).bfloat16()


def test_constant_flow_makes_the_euler_recursion_a_closed_form():
    """A zero head weight leaves flow = head bias b for every input.  The four steps at sigma 1, .75, .5, .25 -> 0
    then give x = noise - b exactly (b = 0.25 and noise on a 1/16 grid: every partial sum is a bf16 number)."""
    P = make_params(CFG, head_weight_scale=0.0, head_bias=0.25)
    noise, ctx = _inputs(2, grid=True)
    trace = []
    out, _ = go.generate(P, CFG, noise, ctx, trace=trace)
    assert len(trace) == 8 and all(torch.all(f == 0.25) for _, _, f in trace)
    assert torch.equal(out, (noise.float() - 0.25).bfloat16())
    # a different schedule: sigma 1 -> .5 -> 0 also integrates to noise - b; a schedule starting at .5 to noise - b/2
    out2, _ = go.generate(P, CFG, noise, ctx, timesteps=(1000.0, 500.0))
    assert torch.equal(out2, out)
    out3, _ = go.generate(P, CFG, noise, ctx, timesteps=(500.0, 250.0))
    assert torch.equal(out3, (noise.float() - 0.125).bfloat16())


def test_cache_bookkeeping_fill_then_roll():
    """local_attn_size 3 frames, sink 1, chunks of 1 frame: the cache fills with chunks 0..2, then every new chunk
    evicts the oldest non-sink chunk.  After chunk c the rows hold [0 | c-1 | c] (token indices), and each layer
    keeps the content of every chunk it ever wrote."""
    P = make_params(CFG)
    noise, ctx = _inputs(5)
    _, caches = go.generate(P, CFG, noise, ctx)
    fs = 16
    for cache in caches:
        st = cache["policy"]
        assert st["global_end"] == 5 * fs and st["local_end"] == 3 * fs
        assert np.array_equal(st["buf"], np.concatenate([np.arange(0, fs), np.arange(3 * fs, 5 * fs)]))
        assert sorted(cache["k"]) == [0, 1, 2, 3, 4] and cache["k"][4].shape == (fs, 2, 128)


def test_chunks_depend_on_the_past_only_and_the_recache_pass_matters():
    P = make_params(CFG)
    noise, ctx = _inputs(4)
    full, _ = go.generate(P, CFG, noise, ctx)
    part, _ = go.generate(P, CFG, noise[:, :2], ctx)
    assert torch.equal(full[:, :2], part)                                  # causal: a prefix run gives the prefix
    other = noise.clone()
    other[:, 3] += 1
    changed, _ = go.generate(P, CFG, other, ctx)
    assert torch.equal(changed[:, :3], full[:, :3]) and not torch.equal(changed[:, 3], full[:, 3])
    # without the timestep-0 pass the cache keeps the K / V of the last denoising forward (noisier input, other
    # timestep embedding): chunk 0 is unaffected, later chunks change
    no_recache, _ = go.generate(P, CFG, noise, ctx, recache=False)
    assert torch.equal(no_recache[:, 0], full[:, 0]) and not torch.equal(no_recache[:, 1:], full[:, 1:])


def test_the_window_forgets_what_rolled_out():
    """With a cache of 3 frames chunk 3 no longer attends chunk 1 (evicted), with a cache of 8 it does: the first
    three chunks agree between the two, chunk 3 differs."""
    P = make_params(CFG)
    noise, ctx = _inputs(4)
    small, _ = go.generate(P, CFG, noise, ctx)
    import dataclasses
    big_cfg = dataclasses.replace(CFG, local_attn_size=8)
    big, _ = go.generate(P, big_cfg, noise, ctx)
    assert torch.equal(small[:, :3], big[:, :3]) and not torch.equal(small[:, 3], big[:, 3])


def test_patch_embedding_and_unpatchify_layouts():
    """The linear-over-patches form equals torch's Conv3d with kernel = stride = patch (fp32 on both sides), and
    the output layout equals the reference's unpatchify einsum 'fhwpqrc->cfphqwr' (causal_model.py:1835-1858)."""
    rng = np.random.default_rng(0)
    C, f, pt, ph, pw, dim = 3, 2, 1, 2, 2, 7
    x = torch.from_numpy(rng.standard_normal((C, f * pt, 4 * ph, 3 * pw)).astype(np.float32))
    wgt = torch.from_numpy(rng.standard_normal((dim, C, pt, ph, pw)).astype(np.float32))
    conv = torch.nn.functional.conv3d(x.unsqueeze(0), wgt, stride=(pt, ph, pw))[0]          # [dim, f, h, w]
    h, w = 4, 3
    patches = x.reshape(C, f, pt, h, ph, w, pw).permute(1, 3, 5, 0, 2, 4, 6).reshape(f * h * w, C * pt * ph * pw)
    lin = patches @ wgt.reshape(dim, -1).T
    assert torch.allclose(lin, conv.flatten(1).T, atol=1e-5)
    c = 5
    tokens = torch.from_numpy(rng.standard_normal((f * h * w, pt * ph * pw * c)).astype(np.float32))
    want = torch.einsum("fhwpqrc->cfphqwr", tokens.view(f, h, w, pt, ph, pw, c)).reshape(c, f * pt, h * ph, w * pw)
    got = tokens.reshape(f, h, w, pt, ph, pw, c).permute(6, 0, 3, 1, 4, 2, 5).reshape(c, f * pt, h * ph, w * pw)
    assert torch.equal(got, want)


def test_sinusoidal_embedding_closed_forms():
    e = go.sinusoidal_embedding_1d(8, torch.tensor([0.0, 1.0]))
    assert torch.equal(e[0], torch.tensor([1.0] * 4 + [0.0] * 4, dtype=torch.float64))
    want = torch.tensor([np.cos(1.0), np.cos(10000 ** -0.25), np.cos(10000 ** -0.5), np.cos(10000 ** -0.75),
                         np.sin(1.0), np.sin(10000 ** -0.25), np.sin(10000 ** -0.5), np.sin(10000 ** -0.75)])
    assert torch.allclose(e[1], want, atol=1e-15)
