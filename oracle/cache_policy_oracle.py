"""Token-level CPU oracle of LongLive's KV-cache policy (TEST INFRASTRUCTURE ONLY: tests import it, the
product never does).

The reference keeps one K and one V buffer of ``kv_cache_size`` token rows per layer plus four scalars
(``global_end_index``, ``local_end_index``, ``pinned_start``, ``pinned_len``).  What a token row holds never
matters to the policy, so this oracle stores in each row the *global index of the token* that was written there
(-1 = never written) and replays the reference's index arithmetic on that array:

* ``attend`` follows ``CausalWanSelfAttention.forward`` (wan_5b/modules/causal_model.py:491-674): the protected
  prefix (global sink, multi-shot pinned region), roll-or-insert decision, the temporary post-roll buffer, and the
  composition of the attended window ([sink] + [pinned] + [local window]); it returns the global indices of the
  attended tokens in attention order together with the reference's ``cache_update_info``.
* ``apply`` follows ``CausalWanModel._apply_cache_updates`` (:1371-1476).
* ``pin_current_chunk`` / ``zero_kv_data`` follow the pipeline's scene-cut handling
  (pipeline/causal_diffusion_inference.py:1017-1043).

Pinned by invariants that a wrong index fails (tests/test_cache_policy.py): the attended tokens of a run without
scene cuts are exactly "first sink frames + the most recent tokens that fit"; the global sink is attended in every
step once written; a pinned chunk that has reached the protected prefix is never evicted; rolling never loses a
token younger than the window; the chunk itself always comes last.  The one behaviour none of these pins is the
reference's use of the not-yet-shifted ``pinned_start`` while it slices the already rolled buffer (:598-606 vs
:651-671): restated as written, **parity unpinned**.
"""
from __future__ import annotations

import numpy as np


def new_state(kv_cache_size: int) -> dict:
    return {"buf": np.full(kv_cache_size, -1, dtype=np.int64), "global_end": 0, "local_end": 0,
            "pinned_start": -1, "pinned_len": 0}


def attend(state: dict, current_start: int, num_new_tokens: int, sink_tokens: int, global_sink_tokens: int,
           max_attention_size: int, local_attn_size: int = 1):
    """One self-attention forward of one layer.  Returns (attended global token indices, update tuple
    (current_end, local_end_index, cache_update_info))."""
    size = len(state["buf"])
    current_end = current_start + num_new_tokens
    new_ids = np.arange(current_start, current_end, dtype=np.int64)
    ps, pl = state["pinned_start"], state["pinned_len"]
    has_pinned = ps >= 0 and pl > 0
    if has_pinned and ps == global_sink_tokens:          # :524-529
        effective_sink = global_sink_tokens + pl
    elif has_pinned:
        effective_sink = global_sink_tokens
    else:
        effective_sink = max(global_sink_tokens, sink_tokens)
    g_end, l_end = state["global_end"], state["local_end"]
    if local_attn_size != -1 and current_end > g_end and num_new_tokens + l_end > size:   # :543-545
        evicted = num_new_tokens + l_end - size
        rolled = l_end - evicted - effective_sink
        local_end = l_end + current_end - g_end - evicted
        local_start = local_end - num_new_tokens
        temp = state["buf"].copy()                                                            # :589-598
        temp[effective_sink:effective_sink + rolled] = \
            state["buf"][effective_sink + evicted:effective_sink + evicted + rolled]
        temp[local_start:local_end] = new_ids
        pinned_shift = evicted if (has_pinned and ps >= effective_sink) else 0                # :606
        info = {"action": "roll_and_insert", "sink_tokens": effective_sink, "num_rolled_tokens": rolled,
                "num_evicted_tokens": evicted, "local_start_index": local_start, "local_end_index": local_end,
                "new_ids": new_ids, "current_end": current_end, "pinned_shift": pinned_shift}
    else:
        local_end = l_end + current_end - g_end                                               # :624-625
        local_start = local_end - num_new_tokens
        temp = state["buf"].copy()
        temp[local_start:local_end] = new_ids
        info = {"action": "direct_insert", "local_start_index": local_start, "local_end_index": local_end,
                "new_ids": new_ids, "current_end": current_end, "pinned_shift": 0}
    window_start = max(0, local_end - max_attention_size)                                     # :674
    prepend_sink = effective_sink > 0 and window_start > 0
    prepend_pinned = has_pinned and ps >= effective_sink and ps < window_start
    if prepend_sink and prepend_pinned:
        local_size = max_attention_size - (effective_sink + pl)
        lws = max(effective_sink, local_end - local_size)
        ids = np.concatenate([temp[:effective_sink], temp[ps:ps + pl], temp[lws:local_end]])
    elif prepend_sink:
        lws = max(effective_sink, local_end - (max_attention_size - effective_sink))
        ids = np.concatenate([temp[:effective_sink], temp[lws:local_end]])
    elif prepend_pinned:
        lws = max(0, local_end - (max_attention_size - pl))
        ids = np.concatenate([temp[ps:ps + pl], temp[lws:local_end]])
    else:
        ids = temp[window_start:local_end]
    return ids, (current_end, local_end, info)


def apply(state: dict, update) -> None:
    current_end, local_end, info = update
    if info is not None:
        buf = state["buf"]
        if info["action"] == "roll_and_insert":
            s, r, e = info["sink_tokens"], info["num_rolled_tokens"], info["num_evicted_tokens"]
            buf[s:s + r] = buf[s + e:s + e + r].copy()
            if info["pinned_shift"] > 0:
                state["pinned_start"] -= info["pinned_shift"]
        buf[info["local_start_index"]:info["local_end_index"]] = info["new_ids"]
    state["global_end"], state["local_end"] = current_end, local_end


def pin_current_chunk(state: dict, chunk_tokens: int, sink_tokens: int) -> None:
    """pipeline:1017-1033: the chunk written last becomes the pinned (multi-shot) sink."""
    state["pinned_start"] = state["local_end"] - chunk_tokens
    state["pinned_len"] = min(sink_tokens, chunk_tokens)


def zero_kv_data(state: dict, current_start_tokens: int, global_sink_tokens: int) -> None:
    """pipeline:1035-1043: forget everything but the global sink before a clean recache."""
    state["local_end"] = global_sink_tokens
    state["global_end"] = current_start_tokens
    state["pinned_start"], state["pinned_len"] = -1, 0
