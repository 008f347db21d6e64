"""CPU oracle of the streaming chunk loop of the NVFP4 generator (TEST INFRASTRUCTURE ONLY).

Restates, on top of the block oracle (``dit_oracle``), the cache-policy oracle (``cache_policy_oracle``) and the
NVFP4 oracle (``nvfp4_oracle``):

* the model forward around the blocks (wan_5b/modules/causal_model.py:1535-1654): patch embedding
  (Conv3d with kernel = stride = patch, :1052-1053, written as the equivalent linear map over patches), time
  embedding (sinusoidal in double, :1554-1564; wan_5b/modules/model.py:15-25), text embedding (:1568-1573), the
  blocks with their KV cache, all cache updates after the last block (:1640-1645, _apply_cache_updates
  :1371-1483: the un-smoothed rotated K and V of the chunk are quantized into the chunk's slot, one amax per
  slot), head (:933-959) and unpatchify (:1835-1858);
* the chunk loop (pipeline/causal_diffusion_inference.py:532-705): per chunk the denoising forwards at the given
  timesteps, each followed by a sampler step, then one forward at timestep 0 that rewrites the chunk's K / V from
  the clean latents (:639-647).  Every forward updates the cache, as in the reference.
  The sampler of the benchmark configuration is the flow-matching Euler step over sigma = t / 1000
  (model/base.py:16-22 gives 1000/750/500/250 for four steps and shift 1): x <- x + (sigma_next - sigma) * flow.

The bf16 ends of the model (embeddings, head) run as torch CPU bf16 operations, the form the reference's eager graph
has; blocks run in numpy through ``dit_oracle.block_forward``.  Per layer the oracle keeps the policy state of
``cache_policy_oracle`` (which token sits in which cache row) and, per written chunk, the dequantized slot content.

Pinning: every component is pinned on its own (see the headers of the three modules); the loop itself is pinned by
closed forms in tests/test_generator_oracle.py (a model whose flow is a known function of its input makes the
Euler recursion a closed form; timestep-0 recache, roll and window bookkeeping are checked against
cache_policy_oracle's invariants; leaving out the recache pass or the roll changes the result).  Against the
reference pipeline itself (needs diffusers / flash_attn, not installed) the composition is **parity unpinned**.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as TF

import cache_policy_oracle as cpo
import dit_oracle
import nvfp4_oracle as o

F32 = np.float32


def _bf(t) -> torch.Tensor:
    return torch.as_tensor(np.asarray(t, dtype=np.float32)).bfloat16() if not isinstance(t, torch.Tensor) else t.bfloat16()


def _np(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def sinusoidal_embedding_1d(dim: int, position: torch.Tensor) -> torch.Tensor:
    """wan_5b/modules/model.py:15-25: cos | sin of position * 10000^(-i/half), in double."""
    half = dim // 2
    position = position.to(torch.float64)
    sinusoid = torch.outer(position, torch.pow(10000, -torch.arange(half).to(position).div(half)))
    return torch.cat([torch.cos(sinusoid), torch.sin(sinusoid)], dim=1)


def new_caches(num_layers: int, kv_cache_size: int) -> list[dict]:
    """Per layer: the policy state, the dequantized content of every chunk written ("k", "v": chunk index ->
    [tokens, heads, head_dim]) and the slot amax it was quantized with ("k_amax", "v_amax")."""
    return [{"policy": cpo.new_state(kv_cache_size), "k": {}, "v": {}, "k_amax": {}, "v_amax": {}}
            for _ in range(num_layers)]


def _gather(content: dict, ids: np.ndarray, blk: int) -> np.ndarray | None:
    """Rows of the cached (dequantized) chunks for the attended global token indices, which come in whole blocks."""
    if ids.size == 0:
        return None
    assert ids.size % blk == 0
    runs = ids.reshape(-1, blk)
    assert np.all(runs[:, 0] % blk == 0) and np.all(np.diff(runs, axis=1) == 1), "attended ranges are whole blocks"
    return np.concatenate([content[int(r[0]) // blk] for r in runs])


def model_forward(P: dict, cfg, x: torch.Tensor, t: torch.Tensor, context: torch.Tensor, caches: list[dict],
                  current_start: int, rule: str = "mse") -> torch.Tensor:
    """One forward of the causal DiT on one chunk.  x bf16 [C_in, F, H, W]; t float [F]; context bf16
    [L, text_dim]; returns the flow prediction bf16 [C_out, F, H, W] and updates ``caches`` in place."""
    pt, ph, pw = cfg.patch_size
    C, Fr, Hh, Ww = x.shape
    f, h, w = Fr // pt, Hh // ph, Ww // pw
    fs, L = h * w, f * h * w
    H, D = cfg.num_heads, cfg.dim // cfg.num_heads
    # patch embedding: Conv3d(kernel = stride = patch) == linear map over flattened patches (c, pt, ph, pw)
    patches = x.reshape(C, f, pt, h, ph, w, pw).permute(1, 3, 5, 0, 2, 4, 6).reshape(L, C * pt * ph * pw)
    xs = TF.linear(patches.bfloat16(), P["patch_embedding.weight"].reshape(cfg.dim, -1), P["patch_embedding.bias"])
    # time embedding and its projection to the six modulation vectors per frame
    e = sinusoidal_embedding_1d(cfg.freq_dim, t.flatten()).bfloat16()
    e = TF.linear(TF.silu(TF.linear(e, P["time_embedding.0.weight"], P["time_embedding.0.bias"])),
                  P["time_embedding.2.weight"], P["time_embedding.2.bias"])                      # [F, dim]
    e0 = TF.linear(TF.silu(e), P["time_projection.1.weight"], P["time_projection.1.bias"]).unflatten(1, (6, cfg.dim))
    # text embedding on the context padded with zero rows to text_len
    ctx = torch.cat([context.bfloat16(), context.new_zeros(cfg.text_len - context.size(0), context.size(1)).bfloat16()])
    ctx = TF.linear(TF.gelu(TF.linear(ctx, P["text_embedding.0.weight"], P["text_embedding.0.bias"]), approximate="tanh"),
                    P["text_embedding.2.weight"], P["text_embedding.2.bias"])
    cos, sin = o.rope_cos_sin(f, h, w, start_frame=current_start // fs, head_dim=D)
    sink_tokens = cfg.sink_size * fs
    max_attn = cfg.local_attn_size * fs
    xn, e0n, ctxn = _np(xs), _np(e0), _np(ctx)
    pending = []
    for li, cache in enumerate(caches):
        ids, update = cpo.attend(cache["policy"], current_start, L, sink_tokens, 0, max_attn)
        cached_ids = ids[:-L]
        assert np.array_equal(ids[-L:], np.arange(current_start, current_start + L)), "the chunk comes last"
        ck, cv = _gather(cache["k"], cached_ids, L), _gather(cache["v"], cached_ids, L)
        xn, rk, v = dit_oracle.block_forward(xn, e0n, ctxn, P["blocks"][li], cos, sin, ck, cv, H, fs, cfg.eps)
        pending.append((update, rk, v))
    # all cache updates after the last block: roll bookkeeping, then quantize-on-write of the chunk's K and V
    for cache, (update, rk, v) in zip(caches, pending):
        cpo.apply(cache["policy"], update)
        for name, val in (("k", rk), ("v", v)):
            vals, sc, am, _ = o.quantize_to_fp4(o.f32_to_bf16(val.reshape(-1, D)), rule)
            cache[name][current_start // L] = o.kv_dequantize(vals, sc, am, rule)[: L * H].reshape(L, H, D)
            cache[name + "_amax"][current_start // L] = float(am)
    # head: LayerNorm without affine, modulated by (head.modulation + e), then the output projection
    hm = _np(P["head.modulation"])[0]                                       # [2, dim]
    en = _np(e)                                                             # [F, dim]
    shift = o.round_bf16(hm[0][None] + en)
    scale1 = o.round_bf16(F32(1) + o.round_bf16(hm[1][None] + en))
    fidx = np.arange(L) // fs
    normed = dit_oracle.layer_norm_affine(xn, np.ones(cfg.dim, F32), np.zeros(cfg.dim, F32), cfg.eps)
    y = o.round_bf16(o.round_bf16(normed * scale1[fidx]) + shift[fidx])
    out = TF.linear(_bf(y), P["head.head.weight"], P["head.head.bias"])     # [L, pt*ph*pw*C_out]
    c = cfg.out_dim
    u = out.reshape(f, h, w, pt, ph, pw, c).permute(6, 0, 3, 1, 4, 2, 5)     # c f pt h ph w pw
    return u.reshape(c, f * pt, h * ph, w * pw)


def generate(P: dict, cfg, noise: torch.Tensor, context: torch.Tensor, timesteps=(1000.0, 750.0, 500.0, 250.0),
             rule: str = "mse", recache: bool = True, trace: list | None = None):
    """noise bf16 [1, F, C, H, W] -> (denoised latents of the same shape, per-layer caches).  ``trace`` (a list)
    receives (chunk, step, flow) for every denoising forward.  ``recache=False`` leaves out the timestep-0 pass
    (used by the tests to show that the pass matters)."""
    _, Fr, C, Hh, Ww = noise.shape
    fs = (Hh // cfg.patch_size[1]) * (Ww // cfg.patch_size[2])
    caches = new_caches(cfg.num_layers, cfg.local_attn_size * fs)
    nb = cfg.num_frame_per_block
    sigmas = [float(t) / 1000.0 for t in timesteps] + [0.0]
    out = torch.empty_like(noise)
    for ci, start in enumerate(range(0, Fr, nb)):
        x = noise[0, start:start + nb].transpose(0, 1).contiguous()           # [C, f, H, W]
        f = x.shape[1]
        for si, t in enumerate(timesteps):
            tt = torch.full((f,), float(t), dtype=torch.float32)
            flow = model_forward(P, cfg, x, tt, context, caches, start * fs, rule)
            if trace is not None:
                trace.append((ci, si, flow))
            x = (x.float() + (sigmas[si + 1] - sigmas[si]) * flow.float()).to(noise.dtype)
        out[0, start:start + f] = x.transpose(0, 1)
        if recache:
            model_forward(P, cfg, x, torch.zeros(f), context, caches, start * fs, rule)
    return out, caches
