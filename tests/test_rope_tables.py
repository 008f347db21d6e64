"""RoPE tables on the CPU: temporal scale and the multi-shot phase offset (host code + oracle)."""
import numpy as np
import torch

import nvfp4_oracle as o
from longlive_amd.utils.rope import build_rope_angles, rope_cos_sin, temporal_angles


ANGLES = build_rope_angles(128)


def test_no_scale_no_offset_is_the_table_slice():
    cos, sin = rope_cos_sin(ANGLES, 3, 4, 5, 7)
    c2, s2 = rope_cos_sin(ANGLES, 3, 4, 5, 7, t_scale=1.0, temporal_offset=0.0)
    assert torch.equal(cos, c2) and torch.equal(sin, s2)
    oc, os_ = o.rope_cos_sin(3, 4, 5, 7)
    assert np.array_equal(cos.numpy(), oc) and np.array_equal(sin.numpy(), os_)


def test_integer_offset_equals_a_later_start_frame():
    a = rope_cos_sin(ANGLES, 4, 2, 3, 5, temporal_offset=9.0)
    b = rope_cos_sin(ANGLES, 4, 2, 3, 14)
    for x, y in zip(a, b):
        assert torch.allclose(x, y, atol=2e-6, rtol=0)
    # and only the temporal columns move
    base = rope_cos_sin(ANGLES, 4, 2, 3, 5)
    nt = 64 - 2 * (64 // 3)
    assert torch.equal(a[0][:, nt:], base[0][:, nt:]) and not torch.allclose(a[0][:, :nt], base[0][:, :nt])


def test_fractional_offset_and_scale_match_the_closed_form_and_the_oracle():
    f, h, w, start, off, ts = 3, 2, 2, 11, 2.5, 0.75
    cos, sin = rope_cos_sin(ANGLES, f, h, w, start, t_scale=ts, temporal_offset=off)
    oc, os_ = o.rope_cos_sin(f, h, w, start, t_scale=ts, temporal_offset=off)
    assert np.allclose(cos.numpy(), oc, atol=2e-6, rtol=0) and np.allclose(sin.numpy(), os_, atol=2e-6, rtol=0)
    nt = 64 - 2 * (64 // 3)
    inv = 1.0 / np.power(10000.0, np.arange(0, 2 * nt, 2, dtype=np.float64) / (2 * nt))
    pos = (np.arange(f) + start + off) * ts
    want = np.cos(pos[:, None] * inv[None, :])
    got = cos.view(f, h, w, -1)[:, 0, 0, :nt].numpy()
    assert np.allclose(got, want, atol=2e-6, rtol=0)


def test_per_frame_offsets():
    per_chunk = torch.tensor([0.0, 1.0, 5.0])
    a = temporal_angles(ANGLES[:, :22], 3, 4, 1.0, per_chunk)
    whole = torch.arange(10, dtype=torch.float64) * 2.0
    b = temporal_angles(ANGLES[:, :22], 3, 4, 1.0, whole)
    inv = ANGLES[1, :22]
    assert torch.allclose(a, (torch.tensor([4.0, 6.0, 11.0], dtype=torch.float64))[:, None] * inv[None, :], atol=1e-12)
    assert torch.allclose(b, (torch.tensor([4.0 + 8.0, 5.0 + 10.0, 6.0 + 12.0], dtype=torch.float64))[:, None] * inv[None, :],
                          atol=1e-12)


def test_a_common_offset_leaves_attention_scores_unchanged():
    """What makes a phase offset harmless inside a scene: RoPE scores depend on position differences only."""
    rng = np.random.default_rng(0)
    q = o.round_bf16(rng.standard_normal((6 * 4, 2, 128)).astype(np.float32))
    k = o.round_bf16(rng.standard_normal((6 * 4, 2, 128)).astype(np.float32))
    def scores(off):
        cs = o.rope_cos_sin(6, 2, 2, 3, temporal_offset=off)
        rq, rk = o.rope_apply(q, *cs), o.rope_apply(k, *cs)
        return np.einsum("qhd,khd->hqk", rq.astype(np.float64), rk.astype(np.float64))
    a, b = scores(0.0), scores(37.25)
    assert np.abs(a - b).max() <= 0.02 * np.abs(a).max()      # bf16 rounding of the rotated vectors only
    cs0, cs1 = o.rope_cos_sin(6, 2, 2, 3), o.rope_cos_sin(6, 2, 2, 3, temporal_offset=37.25)
    mixed = np.einsum("qhd,khd->hqk", o.rope_apply(q, *cs0).astype(np.float64), o.rope_apply(k, *cs1).astype(np.float64))
    assert np.abs(a - mixed).max() > 0.2 * np.abs(a).max()    # different offsets for q and k do change them
