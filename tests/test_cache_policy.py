"""KV-cache policy (sink, global sink, multi-shot pinned region, scene-cut recache) on the CPU.

Two layers: the token-level oracle is pinned by closed forms and invariants of the policy, then the product's
block-level planner (``longlive_amd.utils.kv_cache``), driven through its own update routine with a stand-in for
the quantizer, has to attend exactly the tokens the oracle attends in every step of randomized runs.
"""
import random
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import cache_policy_oracle as cpo

BLK = 4          # tokens per block = tokens per chunk
MAX_BLOCKS = 5
SIZE = BLK * MAX_BLOCKS


def run_oracle(n_chunks, sink, gsink, max_att, cuts=(), clean=False, forwards=2):
    """Streams n_chunks chunks; per chunk `forwards` denoising forwards (updates dropped, as when the dead cache
    writes are skipped... the reference applies them, which rewrites the same rows) and one clean-context forward
    whose update is applied.  Returns the attended ids of every forward and the final state."""
    st = cpo.new_state(SIZE)
    seen = []
    for c in range(n_chunks):
        start = c * BLK
        for _ in range(forwards):
            ids, upd = cpo.attend(st, start, BLK, sink, gsink, max_att)
            cpo.apply(st, upd)
            seen.append((c, ids.copy()))
        if c in cuts and clean:
            cpo.zero_kv_data(st, start, gsink)
        ids, upd = cpo.attend(st, start, BLK, sink, gsink, max_att)
        cpo.apply(st, upd)
        seen.append((c, ids.copy()))
        if c in cuts:
            cpo.pin_current_chunk(st, BLK, sink)
    return seen, st


@pytest.mark.parametrize("sink", [0, BLK, 2 * BLK])
@pytest.mark.parametrize("max_att", [SIZE, SIZE - BLK, SIZE - 2 * BLK])
def test_oracle_without_cuts_is_sink_plus_most_recent(sink, max_att):
    if max_att - sink < 2 * BLK:
        pytest.skip("window too small to hold a chunk and one cached block")
    seen, _ = run_oracle(14, sink, 0, max_att)
    for c, ids in seen:
        end = (c + 1) * BLK
        assert list(ids[-BLK:]) == list(range(end - BLK, end))          # the chunk itself comes last
        if end <= max_att:
            assert list(ids) == list(range(end))                         # everything still fits
        else:
            recent = max_att - sink
            assert list(ids) == list(range(sink)) + list(range(end - recent, end))
        assert len(ids) <= max_att and len(set(ids)) == len(ids)


def test_oracle_global_sink_and_pinned_chunk_survive_every_roll():
    sink = gsink = BLK
    cuts = (3,)
    seen, st = run_oracle(20, sink, gsink, SIZE, cuts=cuts)
    pinned = set(range(3 * BLK, 4 * BLK))
    for c, ids in seen:
        s = set(ids)
        assert set(range(gsink)) <= s                                    # global sink: always attended
        if c > 3:
            assert pinned <= s                                           # the scene's first chunk stays
        assert len(ids) <= SIZE and len(set(ids)) == len(ids)
        end = (c + 1) * BLK
        assert list(ids[-BLK:]) == list(range(end - BLK, end))
    # once the pinned chunk has floated to the front it sits right behind the global sink
    assert st["pinned_start"] == gsink and st["pinned_len"] == BLK
    assert list(st["buf"][gsink:gsink + BLK]) == sorted(pinned)
    # a second scene cut replaces it
    seen, st = run_oracle(20, sink, gsink, SIZE, cuts=(3, 9))
    assert all(set(range(9 * BLK, 10 * BLK)) <= set(ids) for c, ids in seen if c > 9)
    last = seen[-1][1]
    assert not (pinned & set(last))                                      # the first scene's chunk is gone


def test_oracle_clean_recache_forgets_all_but_the_global_sink():
    sink = gsink = BLK
    seen, _ = run_oracle(8, sink, gsink, SIZE, cuts=(5,), clean=True, forwards=0)
    ids = dict(seen)[5]
    assert list(ids) == list(range(gsink)) + list(range(5 * BLK, 6 * BLK))
    ids = dict(seen)[6]
    assert list(ids) == list(range(gsink)) + list(range(5 * BLK, 7 * BLK))


def test_oracle_rolling_never_drops_a_token_younger_than_the_window():
    rnd = random.Random(0)
    for _ in range(50):
        sink = rnd.choice([0, BLK])
        gsink = rnd.choice([0, sink])
        cuts = tuple(sorted(rnd.sample(range(1, 18), rnd.randint(0, 3)))) if gsink else ()
        seen, _ = run_oracle(18, sink, gsink, SIZE, cuts=cuts, forwards=rnd.randint(0, 2))
        for c, ids in seen:
            end = (c + 1) * BLK
            protected = max(sink, gsink) + (BLK if cuts and c > cuts[0] else 0)
            young = range(max(0, end - (SIZE - protected)), end)
            assert set(young) <= set(ids)


# ------------------------------------------------------------------------------------------- the product's planner
class FakeSlot(SimpleNamespace):
    pass


def make_cache():
    def slot():
        return FakeSlot(values=torch.full((1,), -1.0, dtype=torch.float64), scale_factors=torch.zeros(1),
                        amax=torch.zeros(1), scale_rule=None)
    return {"k": [slot() for _ in range(MAX_BLOCKS)], "v": [slot() for _ in range(MAX_BLOCKS)], "quantized": True,
            "block_token_size": BLK, "max_blocks": MAX_BLOCKS, "num_heads": 1,
            "global_end_index": torch.zeros(1, dtype=torch.long), "local_end_index": torch.zeros(1, dtype=torch.long),
            "pinned_start": torch.full((1,), -1, dtype=torch.long), "pinned_len": torch.zeros(1, dtype=torch.long),
            "_global_end": 0, "_local_end": 0, "_pinned_start": -1, "_pinned_len": 0, "_tables": {}}


@pytest.fixture
def kvc(monkeypatch):
    from longlive_amd.utils import kv_cache as mod

    def fake_quantize(block, rule, amax=None, out=None):
        out[0][0] = block[0, 0]          # remember the first token of the block in place of its NVFP4 bytes
    monkeypatch.setattr(mod._native, "quantize", fake_quantize)
    return mod


def planner_ids(kvc, cache, start, sink, gsink, max_att):
    slot_ids, info, local_end = kvc.plan_cache_step(cache, start, BLK, sink, max_att, gsink)
    ids = []
    whole = all(lo == 0 and hi == BLK for _, lo, hi in info["attended_pieces"])
    assert (slot_ids is not None) == whole and (slot_ids is None or list(slot_ids) == [s for s, _, _ in info["attended_pieces"]])
    for s, lo, hi in info["attended_pieces"]:
        first = int(cache["k"][s].values[0])
        ids += list(range(first + lo, first + hi))
    ids += list(range(start, start + BLK))
    new = torch.arange(start, start + BLK, dtype=torch.float64).view(1, BLK, 1, 1).expand(1, BLK, 1, 2)
    info["new_k"], info["new_v"] = new, new
    return ids, (start + BLK, local_end, info)


def test_planner_attends_what_the_oracle_attends(kvc):
    rnd = random.Random(1)
    cfg = SimpleNamespace(scale_rule=SimpleNamespace(value=3))
    runs = steps = 0
    for trial in range(200):
        sink = rnd.choice([0, BLK, 2 * BLK])
        gsink = rnd.choice([0, sink])
        max_att = rnd.choice([SIZE, SIZE, SIZE - BLK, SIZE - BLK // 2, SIZE - BLK - 3])   # windows that end inside a block too
        if max_att - max(sink, gsink) - (BLK if gsink else 0) < 2 * BLK:
            continue
        cuts = tuple(sorted(rnd.sample(range(1, 16), rnd.randint(0, 3)))) if sink else ()
        clean = rnd.random() < 0.4
        forwards = rnd.randint(0, 2)
        st, cache = cpo.new_state(SIZE), make_cache()
        runs += 1
        for c in range(16):
            start = c * BLK
            plan = [False] * forwards + [True]
            for final in plan:
                if final and c in cuts and clean:
                    cpo.zero_kv_data(st, start, gsink)
                    kvc.zero_kv_data([cache], start, gsink)
                want, upd = cpo.attend(st, start, BLK, sink, gsink, max_att)
                try:
                    got, mine = planner_ids(kvc, cache, start, sink, gsink, max_att)
                except NotImplementedError:
                    # only the reference's stale pinned slice may reach into rows the planner cannot name
                    assert st["pinned_start"] >= 0 and upd[2]["action"] == "roll_and_insert"
                    break
                assert got == list(want), (trial, c, sink, gsink, max_att, cuts, clean)
                assert mine[1] == upd[1] and mine[2]["action"] == upd[2]["action"]
                assert mine[2]["pinned_shift"] == upd[2]["pinned_shift"]
                cpo.apply(st, upd)
                kvc.apply_cache_update(cache, mine[0], mine[1], mine[2], cfg)
                steps += 1
                assert cache["_pinned_start"] == st["pinned_start"] == int(cache["pinned_start"])
                assert cache["_local_end"] == st["local_end"] == int(cache["local_end_index"])
            else:
                if c in cuts:
                    cpo.pin_current_chunk(st, BLK, sink)
                    kvc.pin_current_chunk([cache], BLK, sink)
                continue
            break
    assert runs > 100 and steps > 2000


def test_planner_rejects_partial_blocks(kvc):
    cache = make_cache()
    with pytest.raises(NotImplementedError):
        kvc.plan_cache_step(cache, 0, BLK, 2, SIZE)
    with pytest.raises(NotImplementedError):
        kvc.plan_cache_step(cache, 0, BLK - 1, 0, SIZE)
