"""NVFP4 KV cache: allocation, attention over [sink | window | current chunk], roll + insert.

Same cache dictionary as the reference pipeline allocates
(pipeline/causal_diffusion_inference.py:767-813) and the same cache policy as
``CausalWanSelfAttention.forward`` / ``CausalWanModel._apply_cache_updates``
(wan_5b/modules/causal_model.py:491-724, 1371-1483) including the global sink, the multi-shot pinned region
and the scene-cut handling of the pipeline, for whole-block sinks and windows.  Where the
reference dequantizes all slots to bf16, copies the chunk in and calls flash attention, this
module hands the slot list and the chunk's bf16 K/V to one kernel that decodes FP4 tiles on load.
"""
from __future__ import annotations

import torch

from .. import _native
from ..fouroversix import QuantizationConfig, QuantizedTensor, quantize_to_fp4
from .quant import SlotPointerTable, clone_quantized_tensor, copy_quantized_into, dequantize_kv_cache, k_smooth


def initialize_kv_cache(num_layers: int, block_token_size: int, max_blocks: int, num_heads: int, head_dim: int,
                        kv_quant_config: QuantizationConfig, device, dtype=torch.bfloat16) -> list[dict]:
    """One dict per layer; ``k`` / ``v`` are lists of ``max_blocks`` all-zero NVFP4 slots of logical
    shape [block_token_size*num_heads, head_dim]."""
    if head_dim != 128:
        raise ValueError("the KV-cache kernels are built for head_dim 128")
    zero = quantize_to_fp4(torch.zeros(block_token_size * num_heads, head_dim, dtype=dtype, device=device),
                           kv_quant_config)
    cache = []
    for _ in range(num_layers):
        cache.append({
            "k": [clone_quantized_tensor(zero) for _ in range(max_blocks)],
            "v": [clone_quantized_tensor(zero) for _ in range(max_blocks)],
            "quantized": True,
            "block_token_size": block_token_size,
            "max_blocks": max_blocks,
            "num_heads": num_heads,
            "num_filled_blocks": 0,
            # The four scalars of the reference's schema (pipeline/causal_diffusion_inference.py:804-812).  There
            # they live on the device and are published to the host once per forward (utils/wan_5b_wrapper.py:355-366);
            # nothing on the device reads them here, so they are host tensors (an update is then no launch: with
            # device tensors the streaming run issued two small fills per layer and cache write), mirrored as
            # plain ints for the planner.
            "global_end_index": torch.tensor([0], dtype=torch.long),
            "local_end_index": torch.tensor([0], dtype=torch.long),
            "pinned_start": torch.tensor([-1], dtype=torch.long),
            "pinned_len": torch.tensor([0], dtype=torch.long),
            "_global_end": 0,
            "_local_end": 0,
            "_pinned_start": -1,
            "_pinned_len": 0,
            "_tables": {},
            # True: a roll copies slot contents forward like the reference's copy_quantized_into, so that
            # cache["k"][i] keeps its device address for good (utils/quant.py:783-794); False: a roll moves the slot
            # buffers through the lists and copies nothing (see apply_cache_update)
            "stable_slot_addresses": False,
        })
    return cache


_MAX_TABLES = 16


def _tables_for(cache: dict, slot_ids: tuple[int, ...]):
    # keyed by the buffers, not by the positions: a roll moves the buffers through the positions (apply_cache_update),
    # and the handful of arrangements that a streaming run cycles through are each built once
    key = tuple(cache["k"][i].values.data_ptr() for i in slot_ids)
    tables = cache["_tables"]
    entry = tables.pop(key, None)
    if entry is None:
        kt = SlotPointerTable([cache["k"][i] for i in slot_ids])
        vt = SlotPointerTable([cache["v"][i] for i in slot_ids])
        entry = (kt, vt)
        while len(tables) >= _MAX_TABLES:   # scene cuts and varying windows multiply the arrangements: keep the
            tables.pop(next(iter(tables)))  # most recently used ones (dicts keep insertion order)
    tables[key] = entry
    return entry


def plan_cache_step(cache: dict, current_start: int, num_new_tokens: int, sink_tokens: int,
                    max_attention_size: int | None = None, global_sink_tokens: int = 0):
    """Host-side cache policy for one forward of one layer (wan_5b/modules/causal_model.py:491-674): which
    slots are attended, in order, and what ``_apply_cache_updates`` must do afterwards.
    Returns (slot_ids, update_info, local_end).

    The protected prefix of the buffer is the global sink (``global_sink_tokens``, never moves) plus the
    multi-shot pinned region when it sits right behind it; a pinned region elsewhere floats: rolling shifts it
    with the data until it reaches the prefix.  Without a pinned region the prefix is
    ``max(global_sink_tokens, sink_tokens)``.  The attended keys are [prefix] + [floating pinned region, when it
    lies before the window] + [the most recent tokens that fit ``max_attention_size``], the chunk itself last.
    Everything has to fall on block boundaries, since a slot is quantized as a whole."""
    blk = cache["block_token_size"]
    size = cache["max_blocks"] * blk
    g_end, l_end = cache["_global_end"], cache["_local_end"]
    ps, pl = cache.get("_pinned_start", -1), cache.get("_pinned_len", 0)
    current_end = current_start + num_new_tokens
    if num_new_tokens % blk or sink_tokens % blk or global_sink_tokens % blk:
        raise NotImplementedError("the FP4 KV cache works on whole blocks: chunk and sink sizes must be "
                                  f"multiples of block_token_size={blk}")
    has_pinned = ps >= 0 and pl > 0
    if has_pinned and ps == global_sink_tokens:
        effective_sink = global_sink_tokens + pl
    elif has_pinned:
        effective_sink = global_sink_tokens
    else:
        effective_sink = max(global_sink_tokens, sink_tokens)
    if current_end > g_end and num_new_tokens + l_end > size:
        evicted = num_new_tokens + l_end - size
        rolled = l_end - evicted - effective_sink
        local_end = l_end + current_end - g_end - evicted
        local_start = local_end - num_new_tokens
        if evicted % blk or rolled % blk or rolled < 0 or effective_sink % blk:
            raise NotImplementedError("cache roll must move whole blocks")
        info = {"action": "roll_and_insert", "sink_tokens": effective_sink, "num_rolled_tokens": rolled,
                "num_evicted_tokens": evicted, "local_start_index": local_start, "local_end_index": local_end,
                "current_end": current_end,
                "pinned_shift": evicted if (has_pinned and ps >= effective_sink) else 0}
    else:
        evicted = rolled = 0
        local_end = l_end + current_end - g_end
        local_start = local_end - num_new_tokens
        info = {"action": "direct_insert", "local_start_index": local_start, "local_end_index": local_end,
                "current_end": current_end, "pinned_shift": 0}
    if local_start % blk or local_start < 0 or local_end > size:
        raise NotImplementedError("chunks must start on a block boundary of the cache and fit into it")

    def pieces(a: int, b: int) -> list[tuple[int, int, int]]:
        """(slot, first token, end token) pieces that hold rows a..b of the buffer as it will look after the roll."""
        if a < 0 or b > local_start or a > b:
            raise NotImplementedError("attended ranges must lie in the cached part of the buffer (a window shorter than "
                                      "the protected prefix plus the chunk would cut into the chunk itself)")
        out, p = [], a
        while p < b:
            src = p + evicted if effective_sink <= p < effective_sink + rolled else p   # whole blocks move in a roll
            lo = src % blk
            n = min(blk - lo, b - p)
            out.append((src // blk, lo, lo + n))
            p += n
        return out

    window = size if max_attention_size is None else max_attention_size
    window_start = max(0, local_end - window)
    prepend_sink = effective_sink > 0 and window_start > 0
    # the reference slices the rolled buffer with the not yet shifted pinned_start (:651-671)
    prepend_pinned = has_pinned and effective_sink <= ps < window_start
    if prepend_sink and prepend_pinned:
        lws = max(effective_sink, local_end - (window - effective_sink - pl))
        attended = pieces(0, effective_sink) + pieces(ps, ps + pl) + pieces(lws, local_start)
    elif prepend_sink:
        lws = max(effective_sink, local_end - (window - effective_sink))
        attended = pieces(0, effective_sink) + pieces(lws, local_start)
    elif prepend_pinned:
        lws = max(0, local_end - (window - pl))
        attended = pieces(ps, ps + pl) + pieces(lws, local_start)
    else:
        attended = pieces(min(window_start, local_start), local_start)
    # Whole slots go to the attention kernel as they are (it decodes FP4 on load).  A window that does not end on
    # block boundaries (wan_5b/modules/causal_model.py:687-724 slices token rows) attends part of a slot: then the
    # caller dequantizes the slots concerned and attends the bf16 rows, as the reference does for every window.
    info["attended_pieces"] = attended
    whole = all(lo == 0 and hi == blk for _, lo, hi in attended)
    slot_ids = tuple(sl for sl, _, _ in attended) if whole else None
    return slot_ids, info, local_end


def _materialize_pieces(cache: dict, pieces, dtype, device):
    """bf16 K and V rows [n, H, 128] of (slot, first token, end token) pieces, in order: one dequantization launch
    per operand over the slots concerned, then row slices."""
    blk, H = cache["block_token_size"], cache["num_heads"]
    order = sorted({sl for sl, _, _ in pieces})
    pos = {sl: i for i, sl in enumerate(order)}
    kd = dequantize_kv_cache([cache["k"][i] for i in order], len(order), H, blk, dtype, device)[0]
    vd = dequantize_kv_cache([cache["v"][i] for i in order], len(order), H, blk, dtype, device)[0]
    rows = [slice(pos[sl] * blk + lo, pos[sl] * blk + hi) for sl, lo, hi in pieces]
    return torch.cat([kd[r] for r in rows]), torch.cat([vd[r] for r in rows])


def kv_cache_attention(q: torch.Tensor, key_to_cache: torch.Tensor, v: torch.Tensor, cache: dict,
                       current_start: int, sink_tokens: int, softmax_scale: float | None = None,
                       max_attention_size: int | None = None, smoothed_key: torch.Tensor | None = None,
                       amax_out=None, global_sink_tokens: int = 0):
    """Self-attention of one chunk against the FP4 cache.

    q, key_to_cache (RoPE'd, un-smoothed), v: bf16 [1, S, H, 128].  Attends
    [selected FP4 slots | k_smooth(key_to_cache), v] without a mask and returns
    ``(out [1, S, H, 128], (current_end, local_end_index, cache_update_info))`` exactly like the
    reference's attention module, with ``new_k`` / ``new_v`` = the un-smoothed chunk to be written.
    ``smoothed_key`` = k_smooth(key_to_cache) [1, S, H, 128] when the caller has it already (the fused
    norm + RoPE kernel produces it as a second output).  ``amax_out`` (an amax ticket, ``_native.amax_ticket``)
    receives the absolute maximum of ``out``.
    """
    if q.shape[0] != 1:
        raise ValueError("the quantized KV cache holds one sequence (batch size 1)")
    S, H, D = q.shape[1:]
    slot_ids, info, local_end = plan_cache_step(cache, current_start, S, sink_tokens, max_attention_size,
                                                global_sink_tokens)
    info["new_k"], info["new_v"] = key_to_cache, v
    k_new = (k_smooth(key_to_cache) if smoothed_key is None else smoothed_key)[0]
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    rule = cache["k"][0].scale_rule
    if slot_ids is None:   # part of a slot is attended: bf16 rows of the window, then the plain attention kernel
        wk, wv = _materialize_pieces(cache, info["attended_pieces"], q.dtype, q.device)
        out = _native.attention_bf16(q[0].contiguous(), torch.cat([wk, k_new]), torch.cat([wv, v[0]]), scale, amax_out=amax_out)
        return out.unsqueeze(0), (current_start + S, local_end, info)
    if slot_ids:
        kt, vt = _tables_for(cache, slot_ids)
        tables = (kt.values, kt.scales, kt.amax, vt.values, vt.scales, vt.amax)
    else:
        tables = None
    out = _native.kv_attention(q[0].contiguous(), tables, len(slot_ids) * cache["block_token_size"],
                               cache["block_token_size"], rule.max_allowed_e2m1_value(),
                               rule.max_allowed_e4m3_value(), k_new, v[0], scale, amax_out=amax_out)
    return out.unsqueeze(0), (current_start + S, local_end, info)


def kv_cache_update_only(key_to_cache: torch.Tensor, v: torch.Tensor, cache: dict, current_start: int, sink_tokens: int,
                         max_attention_size: int | None = None, global_sink_tokens: int = 0):
    """The ``(current_end, local_end_index, cache_update_info)`` that :func:`kv_cache_attention` (or the relative
    variant) returns beside its output, without the attention: for a layer whose output nobody reads (the last
    layer of a pass that is run only to rewrite the cache)."""
    S = key_to_cache.shape[1]
    _, info, local_end = plan_cache_step(cache, current_start, S, sink_tokens, max_attention_size, global_sink_tokens)
    info["new_k"], info["new_v"] = key_to_cache, v
    return current_start + S, local_end, info


def kv_cache_attention_relative(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cache: dict, current_start: int,
                                sink_tokens: int, rope_fn, softmax_scale: float | None = None,
                                max_attention_size: int | None = None, global_sink_tokens: int = 0):
    """Self-attention of one chunk with *relative* RoPE (wan_5b/modules/causal_model.py:486-487, 716-771): the
    cache holds K without RoPE, and the rotation is applied to the attended window at attention time with the
    frame positions 0, 1, ... of the window itself (sink first), the chunk's queries sitting on its last frames.

    q, k (RMS-normed, no RoPE), v: bf16 [1, S, H, 128]; ``rope_fn(frames, start_frame) -> (cos, sin)`` gives the
    float32 tables of a (frames, h, w) grid.  As in the reference this path materialises the window: the attended
    slots are dequantized to bf16 in one launch, concatenated with the smoothed chunk keys, rotated, and handed
    to the plain bf16 attention kernel.  Returns the same tuple as ``kv_cache_attention``; ``new_k`` is the
    un-rotated ``k``."""
    if q.shape[0] != 1:
        raise ValueError("the quantized KV cache holds one sequence (batch size 1)")
    S, H, D = q.shape[1:]
    frame_seqlen = rope_fn(1, 0)[0].shape[0]
    if S % frame_seqlen or cache["block_token_size"] % frame_seqlen:
        raise ValueError("chunks and cache blocks must hold whole frames")
    slot_ids, info, local_end = plan_cache_step(cache, current_start, S, sink_tokens, max_attention_size,
                                                global_sink_tokens)
    info["new_k"], info["new_v"] = k, v
    keys, values = [k_smooth(k)[0]], [v[0]]
    if info["attended_pieces"]:
        wk, wv = _materialize_pieces(cache, info["attended_pieces"], q.dtype, q.device)
        keys.insert(0, wk)
        values.insert(0, wv)
    window_k, window_v = torch.cat(keys), torch.cat(values)
    if window_k.shape[0] % frame_seqlen:
        raise ValueError("relative RoPE needs an attended window of whole frames")
    window_frames, new_frames = window_k.shape[0] // frame_seqlen, S // frame_seqlen
    from .rope import rope_apply
    roped_k = rope_apply(window_k, *rope_fn(window_frames, 0))
    roped_q = rope_apply(q[0].contiguous(), *rope_fn(new_frames, window_frames - new_frames))
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    out = _native.attention_bf16(roped_q, roped_k, window_v.contiguous(), scale)
    return out.unsqueeze(0), (current_start + S, local_end, info)


def apply_cache_update(cache: dict, current_end: int, local_end_index: int, info: dict | None,
                       kv_quant_config: QuantizationConfig) -> None:
    """Roll whole slots and quantize the chunk's K / V into their slots, in place.

    The reference rolls by copying slot contents forward (causal_model.py:1404-1409) so that slot addresses stay
    put for its CUDA graphs.  The attention kernel here reads the slots through a pointer table, so a roll moves
    the slot buffers through the list instead - the evicted buffers go behind the rolled ones, where the chunk is
    written next - and nothing is copied (18 small device copies per layer and roll otherwise).  Position i of
    ``cache["k"]`` / ``cache["v"]`` holds the same data as after the reference's copies wherever that data is
    meaningful."""
    if info is not None:
        blk = cache["block_token_size"]
        if info["action"] == "roll_and_insert":
            sink_b = info["sink_tokens"] // blk
            ev_b = info["num_evicted_tokens"] // blk
            n_roll = info["num_rolled_tokens"] // blk
            for name in ("k", "v"):
                slots = cache[name]
                if sink_b < 0 or ev_b < 0 or n_roll < 0 or sink_b + ev_b + n_roll > len(slots):
                    raise IndexError(f"roll of {n_roll} blocks behind {sink_b} protected and {ev_b} evicted ones does not fit "
                                     f"a cache of {len(slots)} blocks")
                if cache.get("stable_slot_addresses"):
                    for i in range(n_roll):
                        copy_quantized_into(slots[sink_b + i], slots[sink_b + ev_b + i])
                else:
                    n_slots = len(slots)
                    slots[sink_b:sink_b + ev_b + n_roll] = (slots[sink_b + ev_b:sink_b + ev_b + n_roll]
                                                           + slots[sink_b:sink_b + ev_b])
                    assert len(slots) == n_slots
            if info.get("pinned_shift", 0) > 0:  # a floating pinned region moves with the data (:1437-1443)
                cache["pinned_start"].sub_(info["pinned_shift"])
                cache["_pinned_start"] -= info["pinned_shift"]
        start_blk = info["local_start_index"] // blk
        n_insert = (info["local_end_index"] - info["local_start_index"]) // blk
        rule = kv_quant_config.scale_rule.value
        for bi in range(n_insert):
            blocks, slots, tickets = [], [], []
            for name, new in (("k", info["new_k"]), ("v", info["new_v"])):
                slots.append(cache[name][start_blk + bi])
                blocks.append(new[0, bi * blk:(bi + 1) * blk].reshape(-1, new.shape[-1]))
                # A chunk of one block is quantized as a whole: if its producer left the tensor maximum behind
                # (an amax ticket of the layer's own sink), the quantization takes it from there.
                tickets.append(info.get(f"new_{name}_amax") if n_insert == 1 and new.shape[1] == blk else None)
            outs = [(slot.values, slot.scale_factors, slot.amax) for slot in slots]
            if tickets[0] is not None and tickets[1] is not None and blocks[0].shape == blocks[1].shape:
                _native.quantize_pair(blocks[0], blocks[1], rule, tickets[0], tickets[1], outs[0], outs[1])  # one launch
            else:
                for block, ticket, out in zip(blocks, tickets, outs):
                    _native.quantize(block, rule, amax=ticket, out=out)
    cache["global_end_index"].fill_(current_end)
    cache["local_end_index"].fill_(local_end_index)
    cache["_global_end"] = current_end
    cache["_local_end"] = local_end_index


def pin_current_chunk(kv_cache: list[dict], chunk_tokens: int, sink_tokens: int) -> None:
    """Scene cut with a multi-shot sink: the chunk written last becomes the pinned region of every layer
    (pipeline/causal_diffusion_inference.py:1017-1033).  Nothing is copied; from the next roll on the region
    is protected like the sink once it has floated to the front."""
    for cache in kv_cache:
        start, length = cache["_local_end"] - chunk_tokens, min(sink_tokens, chunk_tokens)
        cache["pinned_start"].fill_(start)
        cache["pinned_len"].fill_(length)
        cache["_pinned_start"], cache["_pinned_len"] = start, length


def zero_kv_data(kv_cache: list[dict], current_start_tokens: int, global_sink_tokens: int) -> None:
    """Scene cut with clean recache: forget everything but the global sink, so that the chunk's clean-context
    forward re-enters it right behind the sink (pipeline/causal_diffusion_inference.py:1035-1043)."""
    for cache in kv_cache:
        cache["local_end_index"].fill_(global_sink_tokens)
        cache["global_end_index"].fill_(current_start_tokens)
        cache["pinned_start"].fill_(-1)
        cache["pinned_len"].zero_()
        cache["_local_end"], cache["_global_end"] = global_sink_tokens, current_start_tokens
        cache["_pinned_start"], cache["_pinned_len"] = -1, 0
