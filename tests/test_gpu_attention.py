"""GPU parity: FP4 KV-cache dequantize, quantize-on-write, fused-dequant attention, RoPE, adaLN, RMSNorm.
Bars: dequant bit-exact; attention <= 2e-2 max-abs on bf16 outputs; RoPE one bf16 ulp; adaLN 3.1e-2."""
import numpy as np
import pytest
import torch

import nvfp4_oracle as o
from helpers import bits_of, u8
from longlive_amd import _native
from longlive_amd.fouroversix import QuantizationConfig, quantize_to_fp4
from longlive_amd.utils import kv_cache as kvc
from longlive_amd.utils.adaln import adaln_modulate
from longlive_amd.utils.quant import dequantize_kv_cache
from longlive_amd.utils.rope import build_rope_angles, rope_apply, rope_cos_sin

pytestmark = pytest.mark.gpu
CFG = QuantizationConfig(scale_rule="mse")


def _randn(shape, seed, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).bfloat16()


def _oracle_slot(t):
    """[T, H, 128] bf16 tensor -> oracle dequantized bf16 values after quantize-on-write."""
    T, H, D = t.shape
    v, s, a, _ = o.quantize_to_fp4(bits_of(t.reshape(-1, D)), "mse")
    return o.kv_dequantize(v, s, a).reshape(T, H, D), (v, s, a)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_kv_dequantize_blocks_bit_exact(gpu, dtype):
    H, T = 4, 96  # 384 rows per slot
    slots, refs = [], []
    for i in range(3):
        t = _randn((T, H, 128), i, scale=1 + i)
        slots.append(quantize_to_fp4(t.reshape(-1, 128).to(gpu), CFG))
        refs.append(_oracle_slot(t)[0])
    got = dequantize_kv_cache(slots, 3, H, T, dtype, gpu)
    assert got.shape == (1, 3 * T, H, 128) and got.dtype == dtype
    ref = np.concatenate(refs)
    if dtype == torch.bfloat16:
        assert np.array_equal(got[0].float().cpu().numpy(), ref)
    else:
        assert np.abs(got[0].cpu().numpy() - ref).max() <= 2 ** -8 * np.abs(ref).max()
        assert np.array_equal(o.round_bf16(got[0].cpu().numpy()), ref)


def test_quantize_on_write_into_slot_is_bit_exact_and_in_place(gpu):
    H, T = 2, 64
    cache = kvc.initialize_kv_cache(1, T, 2, H, 128, CFG, gpu)[0]
    assert not cache["k"][0].values.any() and float(cache["k"][0].amax) == 0.0
    ptrs = [cache["k"][0].values.data_ptr(), cache["k"][0].scale_factors.data_ptr(), cache["k"][0].amax.data_ptr()]
    q, k, v = (_randn((1, T, H, 128), s).to(gpu) for s in (1, 2, 3))
    out, (ce, le, info) = kvc.kv_cache_attention(q, k, v, cache, 0, sink_tokens=T)
    kvc.apply_cache_update(cache, ce, le, info, CFG)
    _, (vals, sc, am) = _oracle_slot(k[0].cpu())
    slot = cache["k"][0]
    assert np.array_equal(u8(slot.values), vals) and np.array_equal(u8(slot.scale_factors), sc)
    assert float(slot.amax.cpu()) == float(am)
    assert ptrs == [slot.values.data_ptr(), slot.scale_factors.data_ptr(), slot.amax.data_ptr()]
    assert int(cache["global_end_index"]) == T and int(cache["local_end_index"]) == T


@pytest.mark.parametrize("Lq,Lk,H", [(64, 64, 1), (128, 200, 2), (100, 333, 3), (257, 130, 2)])
def test_plain_bf16_attention(gpu, Lq, Lk, H):
    q, k, v = _randn((Lq, H, 128), 1), _randn((Lk, H, 128), 2), _randn((Lk, H, 128), 3)
    got = _native.attention_bf16(q.to(gpu), k.to(gpu), v.to(gpu), 128 ** -0.5)
    ref = o.attention(q.float().numpy(), k.float().numpy(), v.float().numpy())
    assert np.abs(got.float().cpu().numpy() - ref).max() <= 2e-2


def test_attention_properties(gpu):
    """Rows of softmax sum to one: with V = ones the output is all ones; a single key returns its value."""
    q = _randn((130, 2, 128), 4).to(gpu)
    k = _randn((77, 2, 128), 5).to(gpu)
    ones = torch.ones(77, 2, 128, dtype=torch.bfloat16, device=gpu)
    out = _native.attention_bf16(q, k, ones, 128 ** -0.5)
    assert (out.float() - 1).abs().max() <= 2 ** -7
    v1 = _randn((1, 2, 128), 6).to(gpu)
    out = _native.attention_bf16(q, k[:1], v1, 128 ** -0.5)
    assert torch.equal(out, v1.expand(130, 2, 128))


@pytest.mark.parametrize("H,T,n_chunks,sink_blocks,max_blocks", [(2, 64, 6, 1, 4), (3, 128, 4, 1, 3), (2, 192, 3, 0, 2), (4, 352, 7, 1, 5)])
def test_cache_streaming_against_oracle(gpu, H, T, n_chunks, sink_blocks, max_blocks):
    """Streams chunks through fill and roll phases; each chunk runs two forwards (the second one
    re-inserts into the same slot, like the clean-context pass).  The oracle keeps a list of
    dequantized slots and applies the reference's policy by hand."""
    cache = kvc.initialize_kv_cache(1, T, max_blocks, H, 128, CFG, gpu)[0]
    ref_slots_k, ref_slots_v = [None] * max_blocks, [None] * max_blocks
    filled = 0
    for c in range(n_chunks):
        for fwd in range(2):
            q, k, v = (_randn((1, T, H, 128), 100 * c + 10 * fwd + s) for s in (1, 2, 3))
            out, (ce, le, info) = kvc.kv_cache_attention(q.to(gpu), k.to(gpu), v.to(gpu), cache, c * T,
                                                         sink_tokens=sink_blocks * T)
            # oracle policy
            if fwd == 0 and filled == max_blocks:  # roll: evict the oldest non-sink slot
                order = list(range(sink_blocks)) + list(range(sink_blocks + 1, max_blocks))
                assert info["action"] == "roll_and_insert"
            elif fwd == 0:
                order = list(range(filled))
            else:
                order = list(range(min(filled, max_blocks) - 1))
            ks = [ref_slots_k[i] for i in order] + [o.k_smooth(k[0].float().numpy())]
            vs = [ref_slots_v[i] for i in order] + [v[0].float().numpy()]
            ref = o.attention(q[0].float().numpy(), np.concatenate(ks), np.concatenate(vs))
            err = np.abs(out[0].float().cpu().numpy() - ref).max()
            assert err <= 2e-2, (c, fwd, err)
            kvc.apply_cache_update(cache, ce, le, info, CFG)
            # oracle cache update
            if fwd == 0 and filled == max_blocks:
                for i in range(sink_blocks, max_blocks - 1):
                    ref_slots_k[i], ref_slots_v[i] = ref_slots_k[i + 1], ref_slots_v[i + 1]
                dst = max_blocks - 1
            elif fwd == 0:
                dst = filled
                filled += 1
            else:
                dst = min(filled, max_blocks) - 1
            ref_slots_k[dst] = _oracle_slot(k[0])[0]
            ref_slots_v[dst] = _oracle_slot(v[0])[0]
        got_k = dequantize_kv_cache(cache["k"], max_blocks, H, T, torch.bfloat16, gpu)[0].float().cpu().numpy()
        for i in range(min(filled, max_blocks)):
            assert np.array_equal(got_k[i * T:(i + 1) * T], ref_slots_k[i]), (c, i)


@pytest.mark.parametrize("window_blocks,clean", [(5, False), (5, True), (4, False), (4, True)])
def test_multi_shot_cache_streaming_against_the_policy_oracle(gpu, window_blocks, clean):
    """Global sink + scene cuts (pinned chunk, optional clean recache) on the FP4 cache: in every forward the
    kernel has to attend exactly the tokens the token-level policy oracle names, with the values the oracle's
    quantize-on-write left for them."""
    import cache_policy_oracle as cpo

    H, T, max_blocks, n_chunks, cuts = 2, 64, 5, 13, (3, 8)
    sink = gsink = T
    cache = kvc.initialize_kv_cache(1, T, max_blocks, H, 128, CFG, gpu)[0]
    st = cpo.new_state(max_blocks * T)
    content = {}   # chunk index -> (dequantized K, dequantized V) as last written
    for c in range(n_chunks):
        for fwd in range(2):
            if fwd == 1 and c in cuts and clean:
                cpo.zero_kv_data(st, c * T, gsink)
                kvc.zero_kv_data([cache], c * T, gsink)
            q, k, v = (_randn((1, T, H, 128), 1000 + 100 * c + 10 * fwd + s) for s in (1, 2, 3))
            ids, upd = cpo.attend(st, c * T, T, sink, gsink, window_blocks * T)
            out, (ce, le, info) = kvc.kv_cache_attention(q.to(gpu), k.to(gpu), v.to(gpu), cache, c * T, sink_tokens=sink,
                                                         max_attention_size=window_blocks * T, global_sink_tokens=gsink)
            chunks = [int(i) // T for i in ids[::T]]
            assert chunks[-1] == c and all(list(ids[j * T:(j + 1) * T]) == list(range(ch * T, (ch + 1) * T))
                                           for j, ch in enumerate(chunks))
            ks = [content[ch][0] for ch in chunks[:-1]] + [o.k_smooth(k[0].float().numpy())]
            vs = [content[ch][1] for ch in chunks[:-1]] + [v[0].float().numpy()]
            ref = o.attention(q[0].float().numpy(), np.concatenate(ks), np.concatenate(vs))
            err = np.abs(out[0].float().cpu().numpy() - ref).max()
            assert err <= 2e-2, (c, fwd, chunks, err)
            assert (le, info["action"], info["pinned_shift"]) == (upd[1], upd[2]["action"], upd[2]["pinned_shift"])
            cpo.apply(st, upd)
            kvc.apply_cache_update(cache, ce, le, info, CFG)
            content[c] = (_oracle_slot(k[0])[0], _oracle_slot(v[0])[0])
        if c in cuts:
            cpo.pin_current_chunk(st, T, sink)
            kvc.pin_current_chunk([cache], T, sink)
        assert int(cache["pinned_start"]) == st["pinned_start"] and int(cache["local_end_index"]) == st["local_end"]
    assert 0 in chunks and 8 in chunks   # the global sink and the last scene's first chunk are still attended
    # the buffer itself: every row up to local_end holds the chunk the oracle says it holds
    got_k = dequantize_kv_cache(cache["k"], max_blocks, H, T, torch.bfloat16, gpu)[0].float().cpu().numpy()
    for b in range(st["local_end"] // T):
        assert np.array_equal(got_k[b * T:(b + 1) * T], content[int(st["buf"][b * T]) // T][0]), b


@pytest.mark.parametrize("window_blocks", [4, 3])
def test_relative_rope_cache_streaming_against_oracle(gpu, window_blocks):
    """Relative RoPE: the cache holds un-rotated K, and every forward rotates the attended window with the frame
    positions of the window itself (queries on its last frames).  Oracle: policy oracle for the token list,
    oracle quantize-on-write for the cached values, oracle RoPE over the window, textbook attention."""
    import cache_policy_oracle as cpo

    H, fh, fw, frames_per_block, max_blocks, n_chunks = 2, 4, 4, 4, 4, 7
    fs = fh * fw
    T = frames_per_block * fs
    sink = T
    angles = build_rope_angles(128)

    def rope_fn(frames, first):
        return rope_cos_sin(angles, frames, fh, fw, first, gpu)

    cache = kvc.initialize_kv_cache(1, T, max_blocks, H, 128, CFG, gpu)[0]
    st = cpo.new_state(max_blocks * T)
    content = {}
    for c in range(n_chunks):
        for fwd in range(2):
            q, k, v = (_randn((1, T, H, 128), 2000 + 100 * c + 10 * fwd + s) for s in (1, 2, 3))
            ids, upd = cpo.attend(st, c * T, T, sink, 0, window_blocks * T)
            out, (ce, le, info) = kvc.kv_cache_attention_relative(q.to(gpu), k.to(gpu), v.to(gpu), cache, c * T, sink, rope_fn,
                                                                  max_attention_size=window_blocks * T)
            chunks = [int(i) // T for i in ids[::T]]
            wk = np.concatenate([content[ch][0] for ch in chunks[:-1]] + [o.k_smooth(k[0].float().numpy())])
            wv = np.concatenate([content[ch][1] for ch in chunks[:-1]] + [v[0].float().numpy()])
            wf = len(chunks) * frames_per_block
            rk = o.rope_apply(wk, *o.rope_cos_sin(wf, fh, fw, 0))
            rq = o.rope_apply(q[0].float().numpy(), *o.rope_cos_sin(frames_per_block, fh, fw, wf - frames_per_block))
            ref = o.attention(rq, rk, wv)
            err = np.abs(out[0].float().cpu().numpy() - ref).max()
            assert err <= 2e-2, (c, fwd, chunks, err)
            assert torch.equal(info["new_k"].cpu(), k)      # what goes into the cache is the un-rotated key
            cpo.apply(st, upd)
            kvc.apply_cache_update(cache, ce, le, info, CFG)
            content[c] = (_oracle_slot(k[0])[0], _oracle_slot(v[0])[0])
    assert chunks == ([0, 4, 5, 6] if window_blocks == 4 else [0, 5, 6])


def test_rope_matches_oracle_bit_exact_and_complex_reference(gpu):
    f, h, w, N = 3, 4, 6, 5
    angles = build_rope_angles()
    cos, sin = rope_cos_sin(angles, f, h, w, start_frame=7, device=gpu)
    oc, os_ = o.rope_cos_sin(f, h, w, start_frame=7)
    assert np.array_equal(cos.cpu().numpy(), oc) and np.array_equal(sin.cpu().numpy(), os_)
    x = _randn((f * h * w + 8, N, 128), 11)
    got = rope_apply(x.to(gpu), cos, sin, seq_len=f * h * w)
    ref = o.rope_apply(x.float().numpy(), oc, os_, seq_len=f * h * w)
    assert np.array_equal(got.float().cpu().numpy(), ref)
    assert torch.equal(got[f * h * w:].cpu(), x[f * h * w:])  # tail rows pass through
    strided = torch.zeros(f * h * w + 8, N, 256, dtype=torch.bfloat16, device=gpu)
    strided[:, :, :128] = x.to(gpu)
    assert torch.equal(rope_apply(strided[:, :, :128], cos, sin, seq_len=f * h * w), got)


def test_rope_benchmark_shape_norm_preservation(gpu):
    f, h, w = 3, 22, 40
    cos, sin = rope_cos_sin(build_rope_angles(), f, h, w, start_frame=12, device=gpu)
    x = _randn((f * h * w, 24, 128), 12).to(gpu)
    y = rope_apply(x, cos, sin)
    n_in = x.float().reshape(-1, 24, 64, 2).norm(dim=-1)
    n_out = y.float().reshape(-1, 24, 64, 2).norm(dim=-1)
    assert ((n_in - n_out).abs() <= 2 ** -7 * n_in + 1e-3).all()


@pytest.mark.parametrize("L,C,fs", [(12, 256, 4), (48, 3072, 16), (6, 1000 - 1000 % 8, 3)])
def test_adaln_against_oracle_and_torch(gpu, L, C, fs):
    F = L // fs
    x = _randn((1, L, C), 13)
    sc, sh = _randn((1, F, 1, C), 14), _randn((1, F, 1, C), 15)
    got = adaln_modulate(x.to(gpu), sc.to(gpu), sh.to(gpu), fs).float().cpu().numpy()[0]
    ref = o.adaln_modulate(x[0].float().numpy(), sc[0, :, 0].float().numpy(), sh[0, :, 0].float().numpy(), fs)
    diff = np.abs(got - ref)
    assert diff.max() <= 3.1e-2 and (diff != 0).mean() < 5e-3
    ln = torch.nn.functional.layer_norm(x.float(), (C,), eps=1e-6).bfloat16()
    eager = (ln.unflatten(1, (F, fs)) * (1 + sc) + sh).flatten(1, 2).float().numpy()[0]
    assert np.abs(got - eager).max() <= 3.1e-2


def test_adaln_strided_modulation_views(gpu):
    """scale / shift are chunk(6) views of one [B, F, 6, C] tensor in the block forward."""
    L, C, fs = 8, 512, 4
    x = _randn((1, L, C), 16).to(gpu)
    e = _randn((1, 2, 6, C), 17).to(gpu)
    parts = e.chunk(6, dim=2)
    got = adaln_modulate(x, parts[1], parts[0], fs)
    ref = adaln_modulate(x, parts[1].contiguous(), parts[0].contiguous(), fs)
    assert torch.equal(got, ref)


def test_rms_norm_against_oracle(gpu):
    x = _randn((50, 3072), 18, scale=3.0)
    w = (1 + 0.1 * torch.randn(3072, generator=torch.Generator().manual_seed(19))).bfloat16()
    got = _native.rms_norm(x.to(gpu), w.to(gpu), 1e-6).float().cpu().numpy()
    ref = o.rms_norm(x.float().numpy(), w.float().numpy())
    diff = np.abs(got - ref)
    assert diff.max() <= 2 ** -5 and (diff != 0).mean() < 5e-3


@pytest.mark.parametrize("L,C,affine", [(37, 256, True), (2640, 3072, True), (10, 4096, False), (5, 1000, True)])
def test_layer_norm_against_oracle_and_torch(gpu, L, C, affine):
    """LayerNorm with weight and bias (the norm ahead of cross-attention): fp32 statistics, one rounding.  Against
    the float64 oracle and against torch's own bf16 layer_norm, each within one bf16 step; the amax it leaves in
    the sink is the maximum of what it wrote."""
    import dit_oracle

    x = _randn((1, L, C), 41, 3.0) + 0.5
    w = (_randn((C,), 42, 0.2) + 1.0) if affine else None
    b = _randn((C,), 43, 0.3) if affine else None
    ticket = _native.amax_ticket(gpu)
    y = _native.layer_norm(x.to(gpu), None if w is None else w.to(gpu), None if b is None else b.to(gpu), 1e-6,
                           amax_out=ticket)
    got = y[0].float().cpu().numpy()
    wn = np.ones(C, np.float32) if w is None else w.float().numpy()
    bn = np.zeros(C, np.float32) if b is None else b.float().numpy()
    ref = dit_oracle.layer_norm_affine(x[0].float().numpy(), wn, bn, 1e-6)
    # one bf16 step at the magnitude of the value, plus the fp32 error of the two terms where they cancel
    step = np.abs(ref) * 2.0 ** -7 + 4e-6 * (np.abs(bn) + 6.0 * np.abs(wn))[None, :]
    assert (np.abs(got - ref) <= step).all()
    assert (got == ref).mean() > 0.98
    t = torch.nn.functional.layer_norm(x.to(gpu), (C,), None if w is None else w.to(gpu), None if b is None else b.to(gpu),
                                       1e-6)[0].float().cpu().numpy()
    assert (np.abs(got - t) <= step).all()
    xq_sink = quantize_to_fp4(y[0], CFG, amax=ticket)
    xq_pass = quantize_to_fp4(y[0], CFG)
    assert float(xq_sink.amax) == float(xq_pass.amax) == np.abs(got).max()
    assert torch.equal(xq_sink.values, xq_pass.values)


def _tile_samples(Lq, H, n_keys):
    """(kind, head, query rows) samples chosen from the launcher's own plan for a shape: a tile that one workgroup
    runs whole, a tile whose parts two or more workgroups compute and one of them combines, and a head's last,
    partly filled group of queries (a "light" tile).  Tile numbering as in the kernel: full tiles first
    (head * full_qtiles + group), the heads' last groups behind them when they are light."""
    from helpers import DIVISION_FIELDS, attention_full_plan, attention_parts

    plan = attention_full_plan(Lq, H, n_keys)
    assert plan["mode"] == 2, plan
    d = {k: plan[k] for k in DIVISION_FIELDS}
    n_full = H * plan["full_qtiles"]

    def rows_of(tile):
        head, group = (tile // plan["full_qtiles"], tile % plan["full_qtiles"]) if tile < n_full else (tile - n_full, plan["full_qtiles"])
        first, last = group * 256, min(Lq, group * 256 + 256)
        # both ends of the tile and the boundary between two waves' queries
        rows = sorted({first, first + 1, first + 31, first + 32, min(first + 127, last - 1), min(first + 128, last - 1), last - 2, last - 1})
        return head, np.array(rows)

    first_split = plan["whole_rounds"] * plan["G"] + plan["extra"]
    samples = []
    if first_split > 0:
        samples.append(("whole", *rows_of(first_split - 1)))   # the last tile that is run whole (an extra one, if any)
        samples.append(("whole", *rows_of(first_split // 2)))
    shared = [t for t in range(plan["split_tiles"]) if len(set(attention_parts(t, d))) == 2]
    assert shared
    for t in (shared[0], shared[len(shared) // 2], shared[-1]):
        tile = first_split + t
        samples.append(("light+shared" if tile >= n_full else "shared", *rows_of(tile)))
    if n_full < H * plan["n_qtiles"]:
        alone = [t for t in range(plan["split_tiles"]) if len(set(attention_parts(t, d))) == 1 and first_split + t >= n_full]
        for t in alone[:1]:
            samples.append(("light", *rows_of(first_split + t)))
    return samples


def _check_samples_against_oracle(out, q, k_all, v_all, samples):
    """fp64-softmax oracle on the sampled query rows (out, q: [Lq, H, 128]; k_all, v_all: [Lk, H, 128])."""
    for kind, h, rows in samples:
        want = o.attention(q[rows, h:h + 1].float().cpu().numpy(), k_all[:, h:h + 1].float().cpu().numpy(),
                           v_all[:, h:h + 1].float().cpu().numpy())
        err = np.abs(out[rows, h:h + 1].float().cpu().numpy() - want).max()
        assert err <= 2e-2, (kind, h, rows, err)


def test_config3_full_size_fused_decode_equals_attention_over_the_dequantized_cache(gpu):
    """Benchmark shape (24 heads, 2640 queries, 4 FP4 slots of 2640 tokens + the bf16 chunk = 13200 keys):
    the kernel that decodes FP4 on load must agree with plain bf16 attention over the cache dequantized by
    ll_kv_dequantize_blocks (a different kernel path), and with the oracle on a sample of queries.  Also a
    row-sum property at full size: with V = const the output is that constant."""
    H, T = 24, 2640
    g = torch.Generator().manual_seed(2)
    cache = kvc.initialize_kv_cache(1, T, 5, H, 128, CFG, gpu)[0]
    for c in range(4):
        q, k, v = (torch.randn(1, T, H, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
        _, (ce, le, info) = kvc.kv_cache_attention(q, k, v, cache, c * T, sink_tokens=T)
        kvc.apply_cache_update(cache, ce, le, info, CFG)
    q, k, v = (torch.randn(1, T, H, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
    out, _ = kvc.kv_cache_attention(q, k, v, cache, 4 * T, sink_tokens=T)
    kd = dequantize_kv_cache(cache["k"], 4, H, T, torch.bfloat16, gpu)[0]
    vd = dequantize_kv_cache(cache["v"], 4, H, T, torch.bfloat16, gpu)[0]
    from longlive_amd.utils.quant import k_smooth
    k_all = torch.cat([kd, k_smooth(k)[0]]).contiguous()
    v_all = torch.cat([vd, v[0]]).contiguous()
    assert k_all.shape == (5 * T, H, 128)
    ref = _native.attention_bf16(q[0].contiguous(), k_all, v_all, 128 ** -0.5)
    assert (out[0].float() - ref.float()).abs().max().item() <= 4e-3  # same bf16 operands, other summation order
    # oracle (fp64 softmax) on the first 16 queries of three heads
    for h in (0, 11, 23):
        want = o.attention(q[0, :16, h:h + 1].float().cpu().numpy(), k_all[:, h:h + 1].float().cpu().numpy(),
                           v_all[:, h:h + 1].float().cpu().numpy())
        assert np.abs(out[0, :16, h:h + 1].float().cpu().numpy() - want).max() <= 2e-2
    # ... and on queries from each kind of tile in the launcher's plan for this shape: tiles run whole by one
    # workgroup, light tiles (queries 2560-2639) computed alone, and light tiles that two workgroups share
    samples = _tile_samples(T, H, 5 * T)
    assert {kind for kind, _, _ in samples} >= {"whole", "light+shared", "light"}
    _check_samples_against_oracle(out[0], q[0], k_all, v_all, samples)
    # rows of the softmax sum to one at full size
    out_c = _native.attention_bf16(q[0].contiguous(), k_all, torch.full_like(v_all, 0.75), 128 ** -0.5)
    assert (out_c.float() - 0.75).abs().max().item() <= 2 ** -7


@pytest.mark.parametrize("H,bts,n_cached,n_new,Lq", [(4, 96, 232, 77, 50), (2, 64, 129, 0, 130), (2, 192, 200, 300, 33),
                                                     (8, 16, 40, 5, 7)])
def test_kernel_accepts_any_number_of_cached_tokens(gpu, H, bts, n_cached, n_new, Lq):
    """The entry point promises any n_cached >= 0: the last slot may be only partly attended, and neither the slot
    size nor n_cached need be a multiple of the kernel's 64- and 128-key tiles.  Checked against the oracle's
    attention over the oracle's dequantization of the attended part of the slots plus the bf16 tail."""
    from longlive_amd.utils.quant import SlotPointerTable
    n_slots = -(-n_cached // bts)
    ks, vs, kq, vq = [], [], [], []
    for i in range(n_slots):
        k, v = _randn((bts, H, 128), 900 + i, 1.0 + 0.25 * i), _randn((bts, H, 128), 950 + i, 0.5 + 0.25 * i)  # amax differs per slot
        ks.append(_oracle_slot(k)[0])
        vs.append(_oracle_slot(v)[0])
        kq.append(quantize_to_fp4(k.reshape(-1, 128).to(gpu), CFG))
        vq.append(quantize_to_fp4(v.reshape(-1, 128).to(gpu), CFG))
    kt, vt = SlotPointerTable(kq), SlotPointerTable(vq)
    tables = [kt.values, kt.scales, kt.amax, vt.values, vt.scales, vt.amax]
    q = _randn((Lq, H, 128), 990)
    k_new = _randn((n_new, H, 128), 991) if n_new else None
    v_new = _randn((n_new, H, 128), 992) if n_new else None
    out = _native.kv_attention(q.to(gpu), tables, n_cached, bts, 6.0, 256.0, k_new.to(gpu) if n_new else None,
                               v_new.to(gpu) if n_new else None, 128 ** -0.5)
    k_all = np.concatenate(ks)[:n_cached]
    v_all = np.concatenate(vs)[:n_cached]
    if n_new:
        k_all = np.concatenate([k_all, k_new.float().numpy()])
        v_all = np.concatenate([v_all, v_new.float().numpy()])
    ref = o.attention(q.float().numpy(), k_all, v_all)
    err = np.abs(out.float().cpu().numpy() - ref).max()
    assert err <= 2e-2, err


@pytest.mark.parametrize("H,bts,n_cached,n_new,Lq,q_scale,k_scale,v_scale", [
    (4, 384, 1023, 24, 1100, 1.0, 2.5, 0.1), (12, 192, 105, 358, 513, 3.0, 0.3, 0.1), (3, 384, 1413, 159, 32, 3.0, 0.3, 1.0),
    (24, 112, 151, 181, 1, 3.0, 1.0, 20.0), (6, 320, 1040, 145, 129, 1.0, 2.5, 20.0), (8, 256, 411, 27, 700, 0.2, 1.0, 20.0)])
def test_error_follows_the_magnitude_of_the_values_attended(gpu, H, bts, n_cached, n_new, Lq, q_scale, k_scale, v_scale):
    """Inputs away from unit scale (sharp and flat softmax, V of 0.1 and 20 with outliers), every work division.
    The 2e-2 bar belongs to unit-scale inputs; what the arithmetic promises in general is relative to the values a
    query attends: the probabilities enter P·V as bf16 (2^-9 each) and the output is bf16 (2^-9), so every output
    lies within 2^-7 of the softmax-weighted mean of |v| from the fp64 result."""
    from longlive_amd.utils.quant import SlotPointerTable
    g = torch.Generator().manual_seed(H * 1000 + Lq)
    def randn(shape, scale):
        x = torch.randn(shape, generator=g) * scale
        return torch.where(torch.rand(shape, generator=g) < 0.002, x * 15, x).bfloat16()
    n_slots = -(-n_cached // bts)
    ks, vs, kq, vq = [], [], [], []
    for i in range(n_slots):
        k, v = randn((bts, H, 128), k_scale * (1 + 0.5 * i)), randn((bts, H, 128), v_scale * (0.5 + 0.5 * i))
        ks.append(_oracle_slot(k)[0])
        vs.append(_oracle_slot(v)[0])
        kq.append(quantize_to_fp4(k.reshape(-1, 128).to(gpu), CFG))
        vq.append(quantize_to_fp4(v.reshape(-1, 128).to(gpu), CFG))
    kt, vt = SlotPointerTable(kq), SlotPointerTable(vq)
    tables = [kt.values, kt.scales, kt.amax, vt.values, vt.scales, vt.amax]
    q, k_new, v_new = randn((Lq, H, 128), q_scale), randn((n_new, H, 128), k_scale), randn((n_new, H, 128), v_scale)
    k_all = np.concatenate([np.concatenate(ks)[:n_cached], k_new.float().numpy()]).astype(np.float64)
    v_all = np.concatenate([np.concatenate(vs)[:n_cached], v_new.float().numpy()]).astype(np.float64)
    qf = q.float().numpy().astype(np.float64)
    ref, mass = np.empty((Lq, H, 128)), np.empty((Lq, H, 128))
    for h in range(H):
        logits = (qf[:, h] @ k_all[:, h].T) * 128 ** -0.5
        prob = np.exp(logits - logits.max(axis=1, keepdims=True))
        prob /= prob.sum(axis=1, keepdims=True)
        ref[:, h], mass[:, h] = prob @ v_all[:, h], prob @ np.abs(v_all[:, h])
    for policy in POLICIES:
        with _native.attention_policy(policy):
            out = _native.kv_attention(q.to(gpu), tables, n_cached, bts, 6.0, 256.0, k_new.to(gpu), v_new.to(gpu), 128 ** -0.5)
        got = out.float().cpu().numpy().astype(np.float64)
        assert np.isfinite(got).all()
        worst = (np.abs(got - ref) / (2.0 ** -7 * mass + 1e-30)).max()
        assert worst <= 1.0, (policy, worst)


def test_release_shape_rolling_window_equals_attention_over_the_dequantized_slots(gpu):
    """Shapes of the reference's released NVFP4 configuration (configs/nvfp4/inference_nvfp4.yaml:3-7: chunks of 8
    frames = 7040 tokens, window 32 frames = 4 blocks, sink 8 frames = 1 block), streamed past the point where
    the window rolls: in chunks 4 and 5 the kernel attends the sink block, the two most recent cached blocks and
    the chunk itself (28160 keys).  Checked against plain bf16 attention over exactly those slots dequantized by
    the separate kernel, and against the oracle's fp64 softmax on a sample of queries of three heads."""
    from longlive_amd.utils.quant import k_smooth
    H, T, blocks = 24, 7040, 4
    g = torch.Generator().manual_seed(7)
    cache = kvc.initialize_kv_cache(1, T, blocks, H, 128, CFG, gpu)[0]
    for c in range(6):
        q, k, v = (torch.randn(1, T, H, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
        slot_ids, _, _ = kvc.plan_cache_step(cache, c * T, T, T, blocks * T)
        out, (ce, le, info) = kvc.kv_cache_attention(q, k, v, cache, c * T, sink_tokens=T, max_attention_size=blocks * T)
        if c >= 4:
            assert info["action"] == "roll_and_insert" and len(slot_ids) == blocks - 1 and slot_ids[0] == 0
            kd = dequantize_kv_cache(cache["k"], blocks, H, T, torch.bfloat16, gpu)[0].view(blocks, T, H, 128)
            vd = dequantize_kv_cache(cache["v"], blocks, H, T, torch.bfloat16, gpu)[0].view(blocks, T, H, 128)
            k_all = torch.cat([kd[i] for i in slot_ids] + [k_smooth(k)[0]]).contiguous()
            v_all = torch.cat([vd[i] for i in slot_ids] + [v[0]]).contiguous()
            assert k_all.shape == (blocks * T, H, 128)
            ref = _native.attention_bf16(q[0].contiguous(), k_all, v_all, 128 ** -0.5)
            assert (out[0].float() - ref.float()).abs().max().item() <= 4e-3
            for h in (0, 13, 23):
                rows = slice(7000, 7016)   # the ragged last query tile (7040 = 55 * 128)
                want = o.attention(q[0, rows, h:h + 1].float().cpu().numpy(), k_all[:, h:h + 1].float().cpu().numpy(),
                                   v_all[:, h:h + 1].float().cpu().numpy())
                assert np.abs(out[0, rows, h:h + 1].float().cpu().numpy() - want).max() <= 2e-2
            if c == 4:
                # queries from every kind of tile of this launch's plan: two whole rounds, 136 full tiles cut
                # into parts for several workgroups, and the 128-query last groups (light, shared as well)
                samples = _tile_samples(T, H, blocks * T)
                assert {kind for kind, _, _ in samples} >= {"whole", "shared", "light+shared"}
                _check_samples_against_oracle(out[0], q[0], k_all, v_all, samples)
            del kd, vd, k_all, v_all, ref
        kvc.apply_cache_update(cache, ce, le, info, CFG)


def test_gate_residual_bit_exact_against_oracle_and_eager(gpu):
    from longlive_amd.utils.adaln import gate_residual
    L, C, fs = 48, 3072, 16
    x, y = _randn((1, L, C), 41), _randn((1, L, C), 42, 3.0)
    e = _randn((1, L // fs, 6, C), 43)          # modulation tensor; the gate is a strided view of it
    gate = e.chunk(6, dim=2)[2]
    got = gate_residual(x.to(gpu), y.to(gpu), e.to(gpu).chunk(6, dim=2)[2], fs)
    want = o.gate_residual(x[0].float().numpy(), y[0].float().numpy(), gate[0, :, 0].float().numpy(), fs)
    assert np.array_equal(got[0].float().cpu().numpy(), want)
    eager = x + (y.unflatten(1, (L // fs, fs)) * gate).flatten(1, 2)
    assert torch.equal(got.cpu(), eager)
    with pytest.raises(ValueError):
        gate_residual(x.to(gpu), y.to(gpu)[:, :, :8], e.to(gpu).chunk(6, dim=2)[2], fs)


def test_fused_norm_rope_equals_the_separate_kernels(gpu):
    """ll_qk_norm_rope against ll_rms_norm followed by ll_rope_apply (bit-exact) and, for the smoothed K,
    against torch's k - k.mean(-1) on the bf16 tensor (same roundings; the fp32 summation order of the mean
    may differ, so a value may move by one bf16 ulp in rare cases)."""
    S, H = 96, 3
    x = _randn((S, H * 128), 51, 2.0).to(gpu)
    w = (1 + 0.1 * torch.randn(H * 128, generator=torch.Generator().manual_seed(52))).bfloat16().to(gpu)
    cos, sin = rope_cos_sin(build_rope_angles(128), 2, 6, 8, 3, gpu)  # 96 rows
    want = rope_apply(_native.rms_norm(x, w, 1e-6).view(S, H, 128), cos, sin)
    got = _native.qk_norm_rope(x, w, 1e-6, cos, sin, H)
    assert torch.equal(got, want)
    got2, smooth = _native.qk_norm_rope(x, w, 1e-6, cos, sin, H, smooth=True)
    assert torch.equal(got2, want)
    eager = want - want.mean(dim=-1, keepdim=True)
    d = (smooth.float() - eager.float()).abs()
    assert float(d.max()) <= 2 ** -7 * float(eager.float().abs().max())
    assert float((d != 0).float().mean()) < 0.01
    # rows beyond seq_len are normalized but not rotated
    part = _native.qk_norm_rope(x, w, 1e-6, cos[:64], sin[:64], H, seq_len=64)
    assert torch.equal(part[:64], want[:64])
    assert torch.equal(part[64:], _native.rms_norm(x, w, 1e-6).view(S, H, 128)[64:])


def test_amax_sink_of_adaln_and_attention_feeds_the_next_quantization(gpu):
    """adaLN and attention leave the absolute maximum of their result in the amax sink; the quantization that
    reads it produces the bytes of a quantization that reduces the tensor itself, also when earlier uses of
    the sink saw larger values."""
    L, C, fs, H = 264, 768, 88, 6
    F = L // fs
    sc, sh = _randn((1, F, 1, C), 61).to(gpu), _randn((1, F, 1, C), 62).to(gpu)
    for scale in (50.0, 1.0, 0.02):
        x = _randn((1, L, C), 63, scale).to(gpu)
        ticket = _native.amax_ticket(gpu)
        y = adaln_modulate(x, sc, sh * scale, fs, amax_out=ticket)
        assert torch.equal(y, adaln_modulate(x, sc, sh * scale, fs))
        a, b = quantize_to_fp4(y[0], CFG, amax=ticket), quantize_to_fp4(y[0], CFG)
        assert float(b.amax) == float(y.abs().max()) and torch.equal(a.amax, b.amax)
        assert torch.equal(a.values, b.values) and np.array_equal(u8(a.scale_factors), u8(b.scale_factors))

        q, k = _randn((L, H, 128), 64).to(gpu), _randn((200, H, 128), 65).to(gpu)
        v = _randn((200, H, 128), 66, scale).to(gpu)
        ticket = _native.amax_ticket(gpu)
        out = _native.attention_bf16(q, k, v, 128 ** -0.5, amax_out=ticket)
        assert torch.equal(out, _native.attention_bf16(q, k, v, 128 ** -0.5))
        a, b = quantize_to_fp4(out.flatten(1), CFG, amax=ticket), quantize_to_fp4(out.flatten(1), CFG)
        assert float(b.amax) == float(out.abs().max()) and torch.equal(a.amax, b.amax)
        assert torch.equal(a.values, b.values) and np.array_equal(u8(a.scale_factors), u8(b.scale_factors))


@pytest.mark.parametrize("S,H", [(50, 24), (7, 40)])  # 24 heads: six groups per lane; 40 heads: the generic width
def test_norm_rope_of_q_and_k_in_one_launch_equals_two_launches(gpu, S, H):
    C = H * 128
    q, k = _randn((S, C), 71, 2.0).to(gpu), _randn((S, C), 72, 2.0).to(gpu)
    wq, wk = (1 + _randn((C,), 73, 0.1)).to(gpu), (1 + _randn((C,), 74, 0.1)).to(gpu)
    cos, sin = rope_cos_sin(build_rope_angles(128), 1, 5, 10, 0, gpu)
    cos, sin = cos[:S].contiguous(), sin[:S].contiguous()
    rq, rk, sk = _native.qk_norm_rope_pair(q, k, wq, wk, 1e-6, cos, sin, H)
    assert torch.equal(rq, _native.qk_norm_rope(q, wq, 1e-6, cos, sin, H))
    one_k, one_s = _native.qk_norm_rope(k, wk, 1e-6, cos, sin, H, smooth=True)
    assert torch.equal(rk, one_k) and torch.equal(sk, one_s)
    with pytest.raises(ValueError):
        _native.qk_norm_rope_pair(q, k[:-1], wq, wk, 1e-6, cos, sin, H)


# --------------------------------------------------------------------------- cached values, bit for bit
# Slot amax values for which the order of the three factors of a cached value is visible in bf16.  A cached
# value is (code * scale) * gs with gs = amax * f32(1/1536) (utils/kernel/kv_dequant_cuda.cu:95-106, 216).
# For the first group, (scale * gs) * code rounds to a different bf16 number for dozens of (scale, code)
# pairs; for the second group the Triton fallback's gs = amax / 1536 (utils/quant.py:753-756) does.  Found by
# enumerating all 2^23 fp32 mantissas of gs on the CPU; the test re-checks both properties before relying on them.
ORDER_SENSITIVE_AMAX = [3.0625, 3.4375, 1.53125, 3.106250047683716, 6.145832538604736, 3.009615421295166]
DIVISION_SENSITIVE_AMAX = [4.34375, 6.640625476837158, 2.0484375953674316, 5.642045021057129]


def _raw_slots(n_slots, rows, amaxes, seed, gpu):
    """Slots of random bytes: every e2m1 code (both zeros included) under every finite e4m3 scale byte."""
    rng = np.random.default_rng(seed)
    host, dev = [], []
    for i in range(n_slots):
        values = rng.integers(0, 256, size=(rows, 64), dtype=np.uint8)
        sb = rng.integers(0, 127, size=(rows, 8), dtype=np.uint8) | (rng.integers(0, 2, size=(rows, 8), dtype=np.uint8) << 7)
        scales = o.to_blocked(sb)
        amax = np.float32(amaxes[i % len(amaxes)])
        host.append((values, scales, amax))
        dev.append((torch.from_numpy(values).to(gpu), torch.from_numpy(scales).to(gpu),
                    torch.tensor([amax], dtype=torch.float32, device=gpu)))
    return host, dev


def _table(dev_slots, gpu):
    t = torch.tensor([[s[j].data_ptr() for s in dev_slots] for j in range(3)], dtype=torch.int64).to(gpu)
    return t[0], t[1], t[2]


@pytest.mark.parametrize("n_cached,n_new", [(384, 0), (360, 0), (64, 0), (384, 100), (200, 128)])
def test_attention_reads_cached_values_bit_for_bit(gpu, n_cached, n_new):
    """The value the attention kernel decodes for a cached token is the bf16 number ll_kv_dequantize_blocks
    returns for it, which is the oracle's (reference: utils/kernel/kv_dequant_cuda.cu:95-106).  Read back
    through the kernel itself: the K slots hold two-hot keys (position t % 64 and 64 + t / 64) and query t is
    the matching two-hot vector, so the score of key t exceeds every other by > 500 in the exponent, the softmax
    is exactly one-hot, and out[t] = 1.0 * V[t] / 1.0.  The V slots are random bytes under slot amax values chosen
    so that any other order of the three factors, or the fallback's divided slot scale, shows in bf16."""
    H, T = 2, 64
    n_slots = (n_cached + T - 1) // T
    amaxes = ORDER_SENSITIVE_AMAX + DIVISION_SENSITIVE_AMAX
    host_v, dev_v = _raw_slots(n_slots, T * H, amaxes, seed=n_cached + n_new, gpu=gpu)
    # keys: token t of the cache -> 64 * (e[t % 64] + e[64 + t // 64]), the same in both heads
    tok = np.arange(n_slots * T)
    kmat = np.zeros((n_slots * T, H, 128), dtype=np.float32)
    kmat[tok, :, tok % 64] = 64.0
    kmat[tok, :, 64 + tok // 64] = 64.0
    k_slots = [quantize_to_fp4(torch.from_numpy(kmat[i * T:(i + 1) * T]).bfloat16().reshape(-1, 128).to(gpu), CFG)
               for i in range(n_slots)]
    dev_k = [(s.values, s.scale_factors.view(torch.uint8), s.amax) for s in k_slots]
    q = torch.from_numpy(kmat[:n_cached]).bfloat16().to(gpu)
    if n_new:  # the chunk's own keys point away from every query, its values are large: any leak would show
        k_new = torch.zeros(n_new, H, 128, dtype=torch.bfloat16, device=gpu)
        k_new[:, :, 127] = -64.0
        v_new = torch.full((n_new, H, 128), 1000.0, dtype=torch.bfloat16, device=gpu)
    else:
        k_new = v_new = None
    tables = _table(dev_k, gpu) + _table(dev_v, gpu)
    out = _native.kv_attention(q, tables, n_cached, T, 6.0, 256.0, k_new, v_new, 128 ** -0.5)
    vt = _table(dev_v, gpu)
    deq = _native.kv_dequantize_blocks(vt[0], vt[1], vt[2], n_slots, H, T, torch.bfloat16, 6.0, 256.0)[0][:n_cached]
    # the sign of a zero does not survive the accumulation (1.0 * -0 + 0 = +0): zeros compare as equal
    ob, db = bits_of(out), bits_of(deq)
    ob[ob == 0x8000] = 0
    db[db == 0x8000] = 0
    assert np.array_equal(ob, db), f"{(ob != db).sum()} of {ob.size} values differ"
    ref = np.concatenate([o.kv_dequantize(v, s, a).reshape(T, H, 128) for v, s, a in host_v])[:n_cached]
    assert np.array_equal(bits_of(deq), o.f32_to_bf16(ref))
    # the inputs do tell the candidate expressions apart
    n_order = n_div = 0
    for v, s, a in host_v:
        if float(a) in ORDER_SENSITIVE_AMAX:
            gs = o.kv_global_scale(a)
            sf = np.repeat(o.e4m3_decode(o.from_blocked(s, (T * H, 8))), 16, axis=1)
            other = o.f32_to_bf16((sf * gs).astype(np.float32) * o.unpack_e2m1(v))
            n_order += int((other != o.f32_to_bf16(o.kv_dequantize(v, s, a))).sum())
        else:
            n_div += int((o.f32_to_bf16(o.kv_dequantize(v, s, a, path="triton")) != o.f32_to_bf16(o.kv_dequantize(v, s, a))).sum())
    if n_slots >= 4:
        assert n_order >= 50
    if n_slots >= len(amaxes) - 3:
        assert n_div >= 10


def test_kv_dequantize_blocks_every_code_and_scale(gpu):
    """ll_kv_dequantize_blocks on random bytes (all codes, all finite scale bytes, both signs) and slot amax values
    sensitive to the factor order, in all three output types, against the oracle."""
    H, T = 4, 96
    host, dev = _raw_slots(5, T * H, ORDER_SENSITIVE_AMAX + DIVISION_SENSITIVE_AMAX, seed=9, gpu=gpu)
    t = _table(dev, gpu)
    ref32 = np.concatenate([o.kv_dequantize(v, s, a, dtype="f32").reshape(T, H, 128) for v, s, a in host])
    got32 = _native.kv_dequantize_blocks(t[0], t[1], t[2], 5, H, T, torch.float32, 6.0, 256.0)[0].cpu().numpy()
    assert np.array_equal(got32.view(np.uint32), ref32.view(np.uint32))
    got16 = _native.kv_dequantize_blocks(t[0], t[1], t[2], 5, H, T, torch.bfloat16, 6.0, 256.0)[0]
    assert np.array_equal(bits_of(got16), o.f32_to_bf16(ref32))
    gotf16 = _native.kv_dequantize_blocks(t[0], t[1], t[2], 5, H, T, torch.float16, 6.0, 256.0)[0]
    assert torch.equal(gotf16.cpu(), torch.from_numpy(ref32).half())


# --------------------------------------------------------------------------- division of a launch between workgroups
POLICIES = ["narrow", "wide", "split"]


@pytest.mark.parametrize("policy", POLICIES)
def test_every_work_division_against_the_oracle(gpu, policy):
    """The three ways a launch is divided between workgroups (one workgroup per 128 queries, per 256 queries, or
    256-query tiles with the key range cut into one equal share per compute unit and the parts combined), forced
    one by one.  Shapes: fewer tiles than compute units, so that under "split" every tile has many parts (a single
    iteration each for Lk = 1500); 320 tiles of two iterations, where a share is the end of one tile, a whole
    tile and the start of a third; 432 tiles of six iterations, which "split" runs as one whole round of 256 and
    the other 176 tiles in equal shares; a last tile with fewer than 32 queries; FP4 slots with a partly attended
    last slot.  Each against the fp64 oracle, and twice for identical bits (the order in which parts arrive must not
    show)."""
    with _native.attention_policy(policy):
        for Lq, Lk, H in [(257, 130, 2), (300, 1500, 3), (700, 900, 2), (2000, 200, 40), (5, 3000, 1), (3000, 700, 36)]:
            q, k, v = _randn((Lq, H, 128), 11), _randn((Lk, H, 128), 12), _randn((Lk, H, 128), 13)
            got = _native.attention_bf16(q.to(gpu), k.to(gpu), v.to(gpu), 128 ** -0.5)
            again = _native.attention_bf16(q.to(gpu), k.to(gpu), v.to(gpu), 128 ** -0.5)
            assert torch.equal(got, again), (policy, Lq, Lk, H)
            ref = o.attention(q.float().numpy(), k.float().numpy(), v.float().numpy())
            err = np.abs(got.float().cpu().numpy() - ref).max()
            assert err <= 2e-2, (policy, Lq, Lk, H, err)
        test_kernel_accepts_any_number_of_cached_tokens(gpu, 4, 96, 232, 77, 50)
        test_kernel_accepts_any_number_of_cached_tokens(gpu, 2, 192, 200, 300, 333)
        test_cache_streaming_against_oracle(gpu, 3, 128, 4, 1, 3)
        test_attention_reads_cached_values_bit_for_bit(gpu, 384, 100)
    assert _native.load().ll_kv_attention_get_policy() == -1


def test_work_divisions_agree_at_the_benchmark_shape_and_leave_the_same_amax(gpu):
    """configs[2] (24 heads, 2640 queries, 13200 keys): the automatic choice is the split of 256-query tiles; its
    output differs from the one-workgroup-per-128-queries result only by the order of fp32 additions, and the
    amax it leaves in the sink is the maximum of its own output."""
    H, T = 24, 2640
    g = torch.Generator().manual_seed(21)
    cache = kvc.initialize_kv_cache(1, T, 5, H, 128, CFG, gpu)[0]
    for c in range(4):
        q, k, v = (torch.randn(1, T, H, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
        _, (ce, le, info) = kvc.kv_cache_attention(q, k, v, cache, c * T, sink_tokens=T)
        kvc.apply_cache_update(cache, ce, le, info, CFG)
    q, k, v = (torch.randn(1, T, H, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
    outs = {}
    for policy in ["auto"] + POLICIES:
        with _native.attention_policy(policy):
            ticket = _native.amax_ticket(gpu)
            outs[policy] = kvc.kv_cache_attention(q, k, v, cache, 4 * T, sink_tokens=T, amax_out=ticket)[0]
            xq = quantize_to_fp4(outs[policy][0].flatten(1), CFG, amax=ticket)
            assert float(xq.amax) == float(outs[policy].float().abs().max())
    assert torch.equal(outs["auto"], outs["split"])
    for policy in ("wide", "split"):
        assert (outs[policy].float() - outs["narrow"].float()).abs().max().item() <= 4e-3
    with pytest.raises(ValueError):
        _native.attention_policy("fastest")
    assert _native.load().ll_kv_attention_set_policy(7) == -1 and b"unknown policy" in _native.load().ll_last_error()


@pytest.mark.parametrize("policy", POLICIES)
@pytest.mark.parametrize("H,n_new,Lq", [(1, 14, 64), (1, 1, 1), (2, 130, 5), (3, 64, 129)])
def test_smallest_launches_under_every_division(gpu, policy, H, n_new, Lq):
    """One tile of one iteration, a single key, a single query: the split division then has a single light unit
    (a plan with no workgroup at all once came out of that) or falls back to whole tiles."""
    q, k, v = _randn((Lq, H, 128), 71), _randn((n_new, H, 128), 72), _randn((n_new, H, 128), 73)
    with _native.attention_policy(policy):
        out = _native.attention_bf16(q.to(gpu), k.to(gpu), v.to(gpu), 128 ** -0.5)
    ref = o.attention(q.float().numpy(), k.float().numpy(), v.float().numpy())
    assert np.abs(out.float().cpu().numpy() - ref).max() <= 2e-2


def test_division_arithmetic_is_the_same_on_device_and_host(gpu):
    """The launcher plans on the host, the kernel walks the plan on the device, the CPU tests check the host side:
    the share boundaries and the holders of every split tile must come out the same on both (64-bit integer
    arithmetic throughout), for the launcher's plans of the benchmark shapes and for a division beyond 32 bits."""
    from helpers import DIVISION_FIELDS, attention_division_on_device, attention_full_plan

    for shape in [(2640, 24, 13200), (7040, 24, 28160), (880, 24, 13200), (3000, 24, 9000), (5, 1, 3000), (1320, 24, 2640)]:
        plan = attention_full_plan(*shape)
        if plan["mode"] != 2:
            continue
        got, host = attention_division_on_device({k: plan[k] for k in DIVISION_FIELDS}, plan["split_tiles"], gpu)
        assert np.array_equal(got, host), shape
    big = dict(G=256, whole_rounds=1, extra=200, n_iter=300001, units=9 * 300001, full_units=2 * 300001, light=12)
    got, host = attention_division_on_device(big, 9, gpu)
    assert np.array_equal(got, host)


@pytest.mark.parametrize("policy", POLICIES)
def test_random_shapes_under_every_division(gpu, policy):
    """Twelve random (heads, slot size, cached tokens, new tokens, queries) combinations per division against the
    oracle: partly attended last slots, no new tokens, no cached tokens, fewer queries than a wave holds."""
    rng = np.random.default_rng(20240607)
    with _native.attention_policy(policy):
        for _ in range(12):
            H = int(rng.choice([1, 2, 4, 8]))
            bts = (128 // H) * int(rng.integers(1, 4))
            n_cached = int(rng.integers(0, 3 * bts + 1))
            n_new = int(rng.integers(0 if n_cached else 1, 300))
            Lq = int(rng.integers(1, 700))
            test_kernel_accepts_any_number_of_cached_tokens(gpu, H, bts, n_cached, n_new, Lq)


def test_launch_on_a_capturing_stream_never_allocates(gpu):
    """A launch recorded into a graph must not allocate, and the clearing of a fresh set of partial-tile records
    must not become a graph node.  On a stream the library has not seen, the automatic choice therefore takes a
    division that needs no memory while the stream is being captured, and an explicit request for the split
    division is refused; once the memory has been reserved on that stream, the recording takes the split division
    and every replay reproduces the eager result bit for bit."""
    Lq, Lk, H = 700, 900, 2
    assert _native.attention_plan(Lq, H, Lk)["division"] == "split"
    q, k, v = (_randn((n, H, 128), s).to(gpu) for n, s in ((Lq, 81), (Lk, 82), (Lk, 83)))
    eager = _native.attention_bf16(q, k, v, 128 ** -0.5)          # split division, memory of the test's stream
    for policy in ("narrow", "wide"):                                # every kernel has run once before a recording
        with _native.attention_policy(policy):
            _native.attention_bf16(q, k, v, 128 ** -0.5)
    ref = o.attention(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy())
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = _native.attention_bf16(q, k, v, 128 ** -0.5)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.abs(out.float().cpu().numpy() - ref).max() <= 2e-2
    assert (out.float() - eager.float()).abs().max().item() <= 4e-3   # another division: other order of additions
    side2 = torch.cuda.Stream(device=gpu)
    side2.wait_stream(torch.cuda.current_stream())
    with _native.attention_policy("split"):
        graph2 = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="captured"):
            with torch.cuda.graph(graph2, stream=side2):
                _native.attention_bf16(q, k, v, 128 ** -0.5)
    del graph2
    torch.cuda.synchronize()
    # with the memory reserved on the stream ahead of the recording, the split division is recorded
    side3 = torch.cuda.Stream(device=gpu)
    side3.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side3):
        _native.attention_reserve(Lq, H, Lk)
    side3.synchronize()
    graph3 = torch.cuda.CUDAGraph()
    with _native.attention_policy("split"), torch.cuda.graph(graph3, stream=side3):
        out3 = _native.attention_bf16(q, k, v, 128 ** -0.5)
    for _ in range(3):
        out3.zero_()
        graph3.replay()
        torch.cuda.synchronize()
        assert torch.equal(out3, eager)
        _native.attention_bf16(q, k, v, 128 ** -0.5)   # eager work between the replays
    # The recorded launches keep the addresses they were recorded with.  When the stream later needs a larger set
    # (the persistent GEMM's partial tiles are larger than the attention's), the recorded one is kept aside, not
    # freed: the graph still replays.
    with torch.cuda.stream(side3):
        _native.gemm_reserve(4096, 4096, 14336)
        _native.attention_bf16(q, k, v, 128 ** -0.5)
    side3.synchronize()
    out3.zero_()
    graph3.replay()
    torch.cuda.synchronize()
    assert torch.equal(out3, eager)
    del graph3
    with torch.cuda.stream(side3):
        _native.attention_release()
    _native.attention_release()   # a stream without memory: nothing to do


@pytest.mark.parametrize("window_tokens,sink_blocks", [(2 * 128 + 40, 1), (3 * 128 - 1, 0), (128 + 64, 0)])
def test_windows_that_end_inside_a_block_against_the_policy_oracle(gpu, window_tokens, sink_blocks):
    """max_attention_size that is not a multiple of the block size (wan_5b/modules/causal_model.py:673-724 slices token
    rows): the local window then begins inside a cached slot.  Token list from the policy oracle, cached values from
    the oracle's quantize-on-write, textbook attention; the cache bytes stay those of whole-block writes."""
    import cache_policy_oracle as cpo

    H, T, max_blocks, n_chunks = 2, 128, 4, 7
    sink = sink_blocks * T
    cache = kvc.initialize_kv_cache(1, T, max_blocks, H, 128, CFG, gpu)[0]
    st = cpo.new_state(max_blocks * T)
    content, partial = {}, 0
    for c in range(n_chunks):
        q, k, v = (_randn((1, T, H, 128), 3000 + 10 * c + s) for s in (1, 2, 3))
        ids, upd = cpo.attend(st, c * T, T, sink, 0, window_tokens)
        out, (ce, le, info) = kvc.kv_cache_attention(q.to(gpu), k.to(gpu), v.to(gpu), cache, c * T, sink_tokens=sink,
                                                     max_attention_size=window_tokens)
        cached = ids[:-T]
        partial += int(any(lo != 0 or hi != T for _, lo, hi in info["attended_pieces"]))
        wk = np.concatenate([content[int(i) // T][0][int(i) % T][None] for i in cached] + [o.k_smooth(k[0].float().numpy())])
        wv = np.concatenate([content[int(i) // T][1][int(i) % T][None] for i in cached] + [v[0].float().numpy()])
        ref = o.attention(q[0].float().numpy(), wk, wv)
        err = np.abs(out[0].float().cpu().numpy() - ref).max()
        assert err <= 2e-2, (c, err)
        cpo.apply(st, upd)
        kvc.apply_cache_update(cache, ce, le, info, CFG)
        content[c] = (_oracle_slot(k[0])[0], _oracle_slot(v[0])[0])
        assert int(cache["local_end_index"]) == st["local_end"]
    assert partial >= 2   # the window did begin inside a slot


def test_roll_with_stable_slot_addresses_copies_like_the_reference(gpu):
    """cache["stable_slot_addresses"] = True: a roll copies slot contents forward (utils/quant.py:783-794), so every
    position of cache["k"] / cache["v"] keeps its buffers for good; outputs and cache contents equal those of the
    default roll, which moves the buffers through the lists."""
    H, T, max_blocks, n_chunks = 2, 64, 3, 6
    caches = [kvc.initialize_kv_cache(1, T, max_blocks, H, 128, CFG, gpu)[0] for _ in range(2)]
    caches[1]["stable_slot_addresses"] = True
    addresses = [[(s.values.data_ptr(), s.scale_factors.data_ptr(), s.amax.data_ptr()) for s in caches[1][n]] for n in ("k", "v")]
    for c in range(n_chunks):
        q, k, v = (_randn((1, T, H, 128), 4000 + 10 * c + s).to(gpu) for s in (1, 2, 3))
        outs = []
        for cache in caches:
            out, (ce, le, info) = kvc.kv_cache_attention(q, k, v, cache, c * T, sink_tokens=T)
            kvc.apply_cache_update(cache, ce, le, info, CFG)
            outs.append(out)
        assert torch.equal(outs[0], outs[1])
        assert addresses == [[(s.values.data_ptr(), s.scale_factors.data_ptr(), s.amax.data_ptr()) for s in caches[1][n]] for n in ("k", "v")]
    for n in ("k", "v"):
        for a, b in zip(caches[0][n], caches[1][n]):
            assert torch.equal(a.values, b.values) and torch.equal(a.scale_factors.view(torch.uint8), b.scale_factors.view(torch.uint8))
            assert torch.equal(a.amax, b.amax)
