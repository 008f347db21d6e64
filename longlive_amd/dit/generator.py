"""Streaming chunk-by-chunk generator with an NVFP4 KV cache.

Mirror of the chunk / denoise loop of the reference pipeline
(pipeline/causal_diffusion_inference.py:532-705): every chunk of ``num_frame_per_block`` latent
frames is denoised with a few flow-matching steps against the cached context and is then run once
more at timestep 0 so that the cache holds the clean chunk's K / V (:639-647).  The cache keeps
``sink_size`` frames plus a sliding window, ``local_attn_size`` frames in total (:775-783).  VAE and
text encoder are outside this path.  Classifier-free guidance (:215, 579-602, 648-657) runs every forward a
second time on the negative prompt against a KV cache of its own and steps with
``uncond + guidance_scale * (cond - uncond)``.

Multi-shot generation (:104-107, 630-665, 974-1043): with ``multi_shot_sink`` the first ``sink_size`` frames of
the stream become a global sink that is never evicted, and the first chunk of every later scene (``scene_cuts``)
is pinned after its clean-context pass, so that the new scene attends its own opening frames instead of the
previous scene's; ``shot_clean_recache`` additionally forgets everything but the global sink before that pass.
``use_relative_rope`` (:149, 316) caches K without RoPE and rotates the attended window by its own frame positions.
``multi_shot_rope_offset`` (:108-112, 439-442, 545-549) shifts the temporal RoPE positions of every scene by
``scene index * offset`` frames, which moves scenes apart in position space.

Two samplers: ``"euler"`` steps the flow prediction over the given timesteps (the fixed 1000/750/500/250
schedule of the benchmark configuration); ``"unipc"`` is the reference pipeline's own choice (:566-612,
892-900): a fresh FlowUniPCMultistepScheduler per chunk with ``len(timesteps)`` steps and ``sample_shift``.
"""
from __future__ import annotations

import torch

from ..fouroversix import ModelQuantizationConfig
from ..utils import kv_cache as kvc
from ..utils.quant import LongLiveQuantizationConfig, quantize_model_with_filter
from ..utils.unipc import FlowUniPCMultistepScheduler
from .model import CausalDiT, DiTConfig


class StreamingGenerator:
    def __init__(self, cfg: DiTConfig, device, timesteps=(1000.0, 750.0, 500.0, 250.0), seed: int = 0,
                 model_quant: dict | None = None, kv_scale_rule: str = "mse", cache_text_kv: bool = True,
                 skip_dead_cache_writes: bool = True, sampler: str = "euler", sample_shift: float = 5.0,
                 multi_shot_sink: bool = False, shot_clean_recache: bool = False,
                 use_relative_rope: bool = False, multi_shot_rope_offset: float = 0.0,
                 guidance_scale: float = 1.0, skip_dead_recache_tail: bool = True) -> None:
        if sampler not in ("euler", "unipc"):
            raise ValueError(f"unknown sampler {sampler!r}")
        self.cfg, self.device = cfg, torch.device(device)
        self.sampler, self.sample_shift = sampler, sample_shift
        self.timesteps = [float(t) for t in timesteps]
        torch.manual_seed(seed)
        with torch.device(self.device):
            model = CausalDiT(cfg)
        model.rope_angles = model.rope_angles.cpu()
        # NVFP4 bring-up in the reference's order (inference.py:341-369): swap the block linears,
        # quantize the weights, drop the bf16 master copies
        model, _ = quantize_model_with_filter(
            model, ModelQuantizationConfig(**(model_quant or {"scale_rule": "mse"})),
            use_default_filtered_modules=True, materialize_for_inference=True, verbose=False)
        self.model = model.eval()
        self.kv_quant_config = LongLiveQuantizationConfig(scale_rule=kv_scale_rule, backend="cuda", type="kv")
        self.model.kv_quant_config = self.kv_quant_config
        self.kv_cache = None
        self.multi_shot_sink, self.shot_clean_recache = multi_shot_sink, shot_clean_recache
        self.multi_shot_rope_offset = float(multi_shot_rope_offset)
        self.guidance_scale = float(guidance_scale)
        self.kv_cache_neg = None
        self.global_sink_size = cfg.sink_size if multi_shot_sink else 0   # :107
        self.model.global_sink_size = self.global_sink_size
        for block in self.model.blocks:                                   # :316
            block.self_attn.use_relative_rope = use_relative_rope
        self.cache_text_kv = cache_text_kv
        self.skip_dead_cache_writes = skip_dead_cache_writes
        # A pass that is run only to rewrite the cache (clean-context pass, context blocks of a continuation) has no
        # reader for its prediction: the last block stops behind its K / V producers and the head is left out.
        self.skip_dead_recache_tail = skip_dead_recache_tail

    def reset_cache(self, frame_seq_length: int) -> None:
        cfg = self.cfg
        block_token_size = cfg.num_frame_per_block * frame_seq_length
        max_blocks = (cfg.local_attn_size * frame_seq_length) // block_token_size
        self.kv_cache = kvc.initialize_kv_cache(cfg.num_layers, block_token_size, max_blocks, cfg.num_heads,
                                                cfg.dim // cfg.num_heads, self.kv_quant_config, self.device)
        self.kv_cache_neg = None
        if self.guidance_scale != 1.0:
            self.kv_cache_neg = kvc.initialize_kv_cache(cfg.num_layers, block_token_size, max_blocks, cfg.num_heads,
                                                        cfg.dim // cfg.num_heads, self.kv_quant_config, self.device)

    @torch.no_grad()
    def generate(self, noise: torch.Tensor, context, on_chunk=None, scene_cuts=(),
                 negative_context: torch.Tensor | None = None,
                 initial_latent: torch.Tensor | None = None, decode_chunk=None,
                 decode_stream: "torch.cuda.Stream | None" = None):
        """noise [1, F, C, H, W] bf16 latents, context [L, text_dim] bf16 (or one such tensor per chunk) ->
        denoised latents of the same shape.  ``on_chunk(index)`` is called after each chunk (timing hooks).
        ``scene_cuts``: indices of the chunks that open a new scene (the reference recognises them by a prefix
        of the chunk's prompt, :974-996); they matter in multi-shot mode only.  ``negative_context`` [L, text_dim]:
        the negative prompt, needed when ``guidance_scale`` is not 1.  ``initial_latent`` [1, F0, C, H, W]: clean
        latents of frames that precede the generated ones (image / video continuation, :375-432): they are run
        through the model at timestep 0 block by block to fill the cache and are returned in front of the generated
        frames; F0 must be a whole number of blocks (the reference's single independent first frame is not
        supported by the block-wise FP4 cache).
        ``decode_chunk(latents [1, C, f, H, W]) -> tensor``: streaming decode (:443-456, 666-683).  Every finished
        chunk is handed to it on ``decode_stream`` (a side stream of default priority, created here when none is
        given) behind an event recorded after the chunk's last denoising step, so that decoding chunk i overlaps the
        clean-context pass of chunk i and the forwards of chunk i + 1; chunks are decoded in order, and the decode
        of chunk i - 1 is waited for before that of chunk i is issued, as the reference's asynchronous VAE path does
        (a decoder that caches features between chunks relies on it).  The return value is then
        ``(latents, [decoded chunks])``; the caller's stream has waited for the last decode."""
        cfg = self.cfg
        _, F, C, H, W = noise.shape
        fs = (H // cfg.patch_size[1]) * (W // cfg.patch_size[2])
        use_cfg = self.guidance_scale != 1.0
        if use_cfg and negative_context is None:
            raise ValueError("guidance_scale != 1 needs negative_context")
        if self.kv_cache is None or (use_cfg and self.kv_cache_neg is None):
            self.reset_cache(fs)
        caches = [self.kv_cache] + ([self.kv_cache_neg] if use_cfg else [])
        xcache_neg = [{"is_init": False} for _ in range(cfg.num_layers)] if (use_cfg and self.cache_text_kv) else None
        nb = cfg.num_frame_per_block
        f0 = 0 if initial_latent is None else initial_latent.shape[1]
        if f0 % nb:
            raise NotImplementedError(f"initial_latent must hold whole blocks of {nb} frames")
        out = noise.new_empty((1, f0 + F) + tuple(noise.shape[2:]))
        first_text = context[0] if isinstance(context, (list, tuple)) else context
        for start in range(0, f0, nb):   # context blocks: clean latents, timestep 0, cache writes only
            x = initial_latent[0, start:start + nb].transpose(0, 1).contiguous()
            out[0, start:start + nb] = initial_latent[0, start:start + nb]
            for cache, text in zip(caches, (first_text, negative_context)):
                self.model(x, torch.zeros((1, nb), device=self.device), text, cache, start * fs, timestep_key=(0.0, nb),
                           cache_only=self.skip_dead_recache_tail)
        # projected text K / V per layer: one prompt per call, so they are computed by the first forward only
        xcache = [{"is_init": False} for _ in range(cfg.num_layers)] if self.cache_text_kv else None
        contexts = list(context) if isinstance(context, (list, tuple)) else None
        scene_cuts = {int(c) for c in scene_cuts}
        shot_index = 0
        self.model.rope_temporal_offset = 0.0
        sigmas = [t / 1000.0 for t in self.timesteps] + [0.0]
        decoded, previous_decode = [], None
        if decode_chunk is not None and decode_stream is None:
            decode_stream = torch.cuda.Stream(device=self.device)
        for ci, src in enumerate(range(0, F, nb)):
            start = f0 + src                                              # position of the chunk in the stream
            x = noise[0, src:src + nb].transpose(0, 1).contiguous()      # [C, f, H, W]
            f = x.shape[1]
            if contexts is not None:
                if ci > 0 and contexts[ci] is not contexts[ci - 1] and xcache is not None:
                    xcache = [{"is_init": False} for _ in range(cfg.num_layers)]  # new prompt: re-project its K / V
                context = contexts[ci]
            if ci > 0 and ci in scene_cuts and self.multi_shot_rope_offset != 0.0:
                shot_index += 1
                self.model.rope_temporal_offset = shot_index * self.multi_shot_rope_offset
            is_scene_cut = self.multi_shot_sink and cfg.sink_size > 0 and ci > 0 and ci in scene_cuts
            if self.sampler == "unipc":
                scheduler = FlowUniPCMultistepScheduler(num_train_timesteps=1000, shift=1)
                scheduler.set_timesteps(len(self.timesteps), device=self.device, shift=self.sample_shift)
                steps = scheduler.timesteps.tolist()
            else:
                scheduler, steps = None, self.timesteps
            for si, t in enumerate(steps):
                tt = torch.full((1, f), float(t), device=self.device, dtype=torch.float32)
                # The K / V a denoising forward would write into the chunk's slot are overwritten by the next
                # forward before anything reads them (the chunk attends its own K / V in bf16), so only the
                # clean-context pass below writes; the cache after the chunk is the same either way.
                flow = self.model(x, tt, context, self.kv_cache, start * fs, crossattn_cache=xcache,
                                  apply_cache_updates=not self.skip_dead_cache_writes, timestep_key=(float(t), f))
                if use_cfg:
                    uncond = self.model(x, tt, negative_context, self.kv_cache_neg, start * fs, crossattn_cache=xcache_neg,
                                        apply_cache_updates=not self.skip_dead_cache_writes, timestep_key=(float(t), f))
                    flow = uncond + self.guidance_scale * (flow - uncond)
                if scheduler is not None:
                    x = scheduler.step(flow, t, x, return_dict=False)[0]
                else:
                    x = (x.float() + (sigmas[si + 1] - sigmas[si]) * flow.float()).to(noise.dtype)
            out[0, start:start + f] = x.transpose(0, 1)
            if decode_chunk is not None:
                chunk_done = torch.cuda.Event()
                chunk_done.record()
                if previous_decode is not None:
                    previous_decode.synchronize()
                with torch.cuda.stream(decode_stream):
                    decode_stream.wait_event(chunk_done)
                    latents = x.unsqueeze(0)
                    latents.record_stream(decode_stream)
                    decoded.append(decode_chunk(latents))
                previous_decode = torch.cuda.Event()
                previous_decode.record(decode_stream)
            # clean-context pass: rewrites this chunk's K / V in the cache
            for cache, text, xc in zip(caches, (context, negative_context), (xcache, xcache_neg)):
                if is_scene_cut and self.shot_clean_recache:
                    kvc.zero_kv_data(cache, start * fs, self.global_sink_size * fs)
                self.model(x, torch.zeros((1, f), device=self.device), text, cache, start * fs, crossattn_cache=xc,
                           timestep_key=(0.0, f), cache_only=self.skip_dead_recache_tail)
                if is_scene_cut:
                    kvc.pin_current_chunk(cache, f * fs, cfg.sink_size * fs)
            if on_chunk is not None:
                on_chunk(ci)
        if decode_chunk is not None:
            torch.cuda.current_stream(self.device).wait_stream(decode_stream)
            return out, decoded
        return out
