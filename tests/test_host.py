"""CPU tests of the host side: the C-ABI library loads and exports every declared symbol, the
configuration / front-end error behaviour mirrors the reference, module swap and cache policy."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from longlive_amd import _native
from longlive_amd.fouroversix import (DataType, FourOverSixLinear, ModelQuantizationConfig, QuantizationConfig,
                                      QuantizedTensor, ScaleRule, fp4_matmul, quantize_model, quantize_to_fp4)
from longlive_amd.utils import kv_cache as kvc
from longlive_amd.utils.quant import LongLiveQuantizationConfig, quantize_model_with_filter


def test_library_loads_and_exports_every_declared_symbol():
    lib = _native.load()
    declared = _native.declared_symbols()
    assert len(declared) >= 13
    for name in declared:
        assert hasattr(lib, name), name
    assert set(declared) == set(_native._SIGNATURES), "ctypes table and header disagree"
    assert lib.ll_version() >= 1
    assert lib.ll_nvfp4_quantize_workspace_floats() == 1024


def test_c_abi_rejects_bad_arguments_without_touching_the_gpu():
    lib = _native.load()
    assert lib.ll_nvfp4_quantize(None, 1, 1, 1, 3, None, None, None, 0, None, None) == -1
    assert b"null pointer" in lib.ll_last_error()
    assert lib.ll_nvfp4_gemm_tnt(None, None, None, None, None, None, None, 1.0, 1.0, 1, 1, 128, 128, 64, None, 1,
                                 None, None) == -1
    assert lib.ll_rope_apply(None, 1, 1, 16, 16, 16, None, None, 1, None, None) == -1
    assert lib.ll_nvfp4_gemm_tnt_fused(None, None, None, None, None, None, None, 1.0, 1.0, 1, 1, 128, 128, 64, None,
                                       1, None, None) == -1
    assert b"null epilogue" in lib.ll_last_error()
    assert lib.ll_nvfp4_quantize_from_sink(None, 1, 1, 1, 3, None, None, None, None, None) == -1
    assert b"null amax sink" in lib.ll_last_error()
    import ctypes
    gated = _native.GemmEpilogue(None, 0, 1 << 20, 4, 8, None, 0, _native.AmaxSinkStruct(None, 0))
    assert lib.ll_nvfp4_gemm_tnt_fused(None, None, None, None, None, None, None, 1.0, 1.0, 1, 1, 128, 128, 64, None,
                                       1, ctypes.byref(gated), None) == -1
    assert b"a gate needs a residual" in lib.ll_last_error()
    assert ctypes.sizeof(_native.GemmEpilogue) == 80 and ctypes.sizeof(_native.AmaxSinkStruct) == 24
    assert ctypes.sizeof(_native.GemmProduct) == 88
    assert lib.ll_amax_epoch_advance(None, 1, None, None) == -1 and b"epoch_offset" in lib.ll_last_error()


def test_one_launch_entry_points_check_their_arguments_before_touching_the_gpu():
    """ll_adaln_quantize / ll_layer_norm_quantize / ll_nvfp4_quantize_pair_from_sinks: null pointers, a missing amax
    sink, and shapes the kernels do not take are answered on the host (LL_EINVAL = -1, LL_ENOSUP = -3)."""
    import ctypes
    lib = _native.load()
    buf = (ctypes.c_uint8 * 4096)()                     # aligned host memory: only its address is looked at
    ptr = ctypes.addressof(buf) + (-ctypes.addressof(buf)) % 256
    sink = _native.AmaxSinkStruct(ptr, 1, None)
    assert lib.ll_adaln_quantize(None, 1, 16, 64, None, None, 0, 0, 0, 0, 16, 1e-6, 1, 3, None, None, None, None, 64, None) == -1
    assert b"null pointer" in lib.ll_last_error()
    assert lib.ll_adaln_quantize(ptr, 1, 16, 64, ptr, ptr, 0, 0, 0, 0, 16, 1e-6, 1, 3, ptr, ptr, ptr, None, 64, None) == -1
    assert b"amax sink" in lib.ll_last_error()
    assert lib.ll_adaln_quantize(ptr, 1, 16, 64, ptr, ptr, 0, 0, 0, 0, 5, 1e-6, 1, 3, ptr, ptr, ptr, ctypes.byref(sink), 64, None) == -1
    assert b"bad shape" in lib.ll_last_error()            # L is not a whole number of frames
    assert lib.ll_adaln_quantize(ptr, 1, 16, 96, ptr, ptr, 0, 0, 0, 0, 16, 1e-6, 1, 3, ptr, ptr, ptr, ctypes.byref(sink), 64, None) == -3
    assert b"multiple of 64" in lib.ll_last_error()
    assert lib.ll_layer_norm_quantize(ptr, 16, 4096, None, None, 1e-6, 3, ptr, ptr, ptr, ctypes.byref(sink), 64, None) == -3
    assert lib.ll_layer_norm_quantize(ptr, 16, 64, None, None, 1e-6, 9, ptr, ptr, ptr, ctypes.byref(sink), 64, None) == -1
    assert b"scale rule" in lib.ll_last_error()
    assert lib.ll_nvfp4_quantize_pair_from_sinks(ptr, ptr, 16, 64, 64, 3, ptr, ptr, ptr, ptr, ptr, ptr, ctypes.byref(sink),
                                                 ctypes.byref(sink), None) == -1
    assert b"outputs of their own" in lib.ll_last_error()
    assert lib.ll_nvfp4_quantize_pair_from_sinks(ptr, ptr, 16, 64, 64, 3, ptr, ptr + 256, ptr, ptr + 256, ptr, ptr + 256,
                                                 None, ctypes.byref(sink), None) == -1
    assert b"null amax sink" in lib.ll_last_error()


def test_noalloc_quantize_refuses_inputs_beyond_its_limit_before_touching_the_gpu():
    lib = _native.load()
    limit = lib.ll_nvfp4_quantize_noalloc_max_elements()
    assert limit == 1 << 32
    assert lib.ll_nvfp4_quantize_noalloc(None, limit // 64 + 1, 64, 64, 3, None, None, None, None) == -1
    assert b"exceed the limit" in lib.ll_last_error()
    assert lib.ll_nvfp4_quantize_noalloc(None, 0, 64, 64, 3, None, None, None, None) == -1


def test_amax_ticket_misuse_is_refused_on_the_host():
    """All tickets of a device share one sink buffer.  A quantization may consume a ticket only while that
    ticket's producer launch is the latest one on the sink; the host bookkeeping refuses anything else instead of
    letting the kernel quantize against another tensor's (or no) maximum."""
    cpu = torch.device("cpu")
    a = _native.amax_ticket(cpu)
    with pytest.raises(RuntimeError, match="not the latest producer"):   # never handed to a producer
        _native._check_consumer(a)
    _native._sink_struct(a)                                              # producer launch with ticket a
    _native._check_consumer(a)                                           # its consumer: fine, also repeatedly
    _native._check_consumer(a)
    b = _native.amax_ticket(cpu)
    assert b.epoch == a.epoch + 1 and b.parts is a.parts
    _native._check_consumer(a)                                           # issuing a ticket alone changes nothing
    _native._sink_struct(b)                                              # another producer launches in between
    with pytest.raises(RuntimeError, match="not the latest producer"):
        _native._check_consumer(a)
    _native._check_consumer(b)
    assert _native._sink_struct(None).parts is None
    with pytest.raises(TypeError):
        _native._sink_struct(object())


def test_patch_embedding_as_matrix_product_equals_the_convolution():
    """CausalDiT.patch_embed runs the Conv3d with kernel = stride = patch (wan_5b/modules/causal_model.py:1052-1053)
    as one matrix product over flattened patches; fp32 on the CPU it must reproduce torch's convolution."""
    from longlive_amd.dit.model import CausalDiT, DiTConfig

    torch.manual_seed(0)
    cfg = DiTConfig(dim=64, ffn_dim=128, num_heads=1, num_layers=0, in_dim=5, out_dim=5, text_dim=16, text_len=4)
    m = CausalDiT(cfg)
    x = torch.randn(5, 3, 8, 12)
    tokens, grid = m.patch_embed(x)
    conv = m.patch_embedding(x.unsqueeze(0))
    assert grid == tuple(conv.shape[2:]) == (3, 4, 6)
    assert torch.allclose(tokens, conv.flatten(2).transpose(1, 2), atol=1e-6)


def test_scale_rule_tables():
    assert [ScaleRule(r).cuda_id() for r in ("static_6", "static_4", "mae", "mse", "abs_max")] == [0, 1, 2, 3, 4]
    assert ScaleRule.mse.max_allowed_e4m3_value() == 256 and ScaleRule.static_4.max_allowed_e2m1_value() == 4
    assert DataType.nvfp4.block_size() == 16 and DataType.nvfp4.scale_dtype() == torch.float8_e4m3fn
    cfg = QuantizationConfig(scale_rule="mae", backend="cuda")
    assert cfg.scale_rule is ScaleRule.mae and cfg.dtype is DataType.nvfp4


@pytest.mark.parametrize("kwargs", [dict(dtype="mxfp4", scale_rule="static_6"), dict(round_style="stochastic"),
                                    dict(rht=True), dict(block_scale_2d=True), dict(transpose=True)])
def test_unsupported_quantization_options_raise_value_error(kwargs):
    with pytest.raises(ValueError, match="does not support"):
        quantize_to_fp4(torch.zeros(128, 64, dtype=torch.bfloat16), QuantizationConfig(**kwargs))


def test_front_ends_fail_loudly_off_gpu():
    x = torch.zeros(128, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU only"):
        quantize_to_fp4(x)
    with pytest.raises(ValueError, match="2-D"):
        quantize_to_fp4(torch.zeros(2, 128, 64, dtype=torch.bfloat16))
    qt = QuantizedTensor(torch.zeros(128, 32, dtype=torch.uint8), torch.zeros(128 * 4, dtype=torch.float8_e4m3fn),
                         torch.zeros(1), "nvfp4", (128, 64), "mse")
    assert qt.padded_shape == (128, 64)
    other = QuantizedTensor(torch.zeros(128, 64, dtype=torch.uint8), torch.zeros(128 * 8, dtype=torch.float8_e4m3fn),
                            torch.zeros(1), "nvfp4", (128, 128), "mse")
    with pytest.raises(ValueError, match="same inner dimension"):
        fp4_matmul(qt, other)
    with pytest.raises(ValueError, match="out_dtype"):
        fp4_matmul(qt, qt, out_dtype=DataType.float16)


def test_quantized_tensor_pads_and_blocks_2d_scales():
    values = torch.arange(100 * 24, dtype=torch.int64).remainder(251).to(torch.uint8).reshape(100, 24)
    scales = torch.arange(100 * 3).remainder(120).to(torch.uint8).reshape(100, 3)
    qt = QuantizedTensor(values, scales, torch.ones(1), DataType.nvfp4, (100, 48), ScaleRule.mse)
    assert qt.padded_shape == (128, 64) and qt.values.shape == (128, 32) and qt.scale_factors.shape == (512,)
    assert torch.equal(qt.values[:100, :24], values) and not qt.values[100:].any() and not qt.values[:, 24:].any()
    from longlive_amd.fouroversix.quantize.utils import from_blocked

    back = from_blocked(qt.scale_factors.view(torch.uint8), (128, 4))
    assert torch.equal(back[:100, :3], scales) and not back[100:].any() and not back[:, 3:].any()
    with pytest.raises(ValueError, match="scale factors"):  # 1-D scales are taken as already blocked
        QuantizedTensor(torch.zeros(128, 32, dtype=torch.uint8), torch.zeros(300, dtype=torch.float8_e4m3fn),
                        torch.ones(1), DataType.nvfp4, (100, 48), ScaleRule.mse)


class _Tiny(nn.Module):
    def __init__(self):
        super().__init__()
        self.text_embedding = nn.Sequential(nn.Linear(64, 64), nn.GELU(), nn.Linear(64, 64))
        self.blocks = nn.ModuleList([nn.ModuleDict(dict(q=nn.Linear(64, 64), norm_q=nn.LayerNorm(64),
                                                        ffn=nn.Sequential(nn.Linear(64, 128), nn.GELU(), nn.Linear(128, 64))))
                                     for _ in range(2)])
        self.head = nn.ModuleDict(dict(head=nn.Linear(64, 16)))


def test_quantize_model_with_filter_swaps_only_unfiltered_linears():
    model, matched = quantize_model_with_filter(_Tiny(), {"scale_rule": "mse"}, use_default_filtered_modules=True,
                                                verbose=False)
    assert isinstance(model.blocks[0]["q"], FourOverSixLinear) and isinstance(model.blocks[1]["ffn"][2], FourOverSixLinear)
    assert type(model.text_embedding[0]) is nn.Linear and type(model.head["head"]) is nn.Linear
    assert "head.head" in matched and "blocks.0.norm_q" in matched
    lin = model.blocks[0]["q"]
    assert lin.weight.dtype == torch.bfloat16
    sd = lin.state_dict()
    assert sd["quantized_weight_values"].shape == (64, 32) and sd["quantized_weight_values"].dtype == torch.uint8
    assert sd["quantized_weight_scale_factors"].shape == (64 * 64 // 16,)
    assert sd["quantized_weight_scale_factors"].dtype == torch.float8_e4m3fn
    assert sd["quantized_weight_amax"].shape == (1,) and sd["quantized_weight_metadata"].shape == (4,)
    with pytest.raises(TypeError):
        quantize_model_with_filter(_Tiny(), quant_config=3, verbose=False)
    with pytest.raises(ValueError, match="filter_profile"):
        quantize_model_with_filter(_Tiny(), use_default_filtered_modules=True, filter_profile="nope", verbose=False)
    cfg = ModelQuantizationConfig(modules_to_not_convert=["blocks.0.q"])
    m2 = _Tiny()
    quantize_model(m2, cfg)
    assert type(m2.blocks[0]["q"]) is nn.Linear and isinstance(m2.blocks[1]["q"], FourOverSixLinear)


def test_longlive_quantization_config_type_field():
    assert LongLiveQuantizationConfig(scale_rule="mse", backend="cuda", type="kv").type == "kv"
    with pytest.raises(ValueError, match="Unknown quantization type"):
        LongLiveQuantizationConfig(type="bogus")


def test_install_as_fouroversix_alias():
    import longlive_amd

    longlive_amd.install_as_fouroversix()
    from fouroversix import QuantizedTensor as Q2  # noqa: PLC0415
    from fouroversix.quantize.quantized_tensor import from_blocked  # noqa: F401, PLC0415

    assert Q2 is QuantizedTensor


def _fake_cache(blk, max_blocks):
    return {"block_token_size": blk, "max_blocks": max_blocks, "_global_end": 0, "_local_end": 0}


def test_cache_policy_fill_then_roll_matches_reference_numbers():
    """Benchmark geometry: block 2640 tokens, 5 slots, sink = 1 block
    (wan_5b/modules/causal_model.py:548-555, 623-626 evaluated by hand)."""
    blk = 2640
    cache = _fake_cache(blk, 5)
    for chunk in range(5):  # fill phase: direct insert at local_end, attends slots [0, chunk)
        for forward in range(2):  # the second forward of a chunk re-inserts into the same slot
            slots, info, local_end = kvc.plan_cache_step(cache, chunk * blk, blk, blk, 5 * blk)
            assert info["action"] == "direct_insert" and slots == tuple(range(chunk))
            assert (info["local_start_index"], local_end) == (chunk * blk, (chunk + 1) * blk)
            cache["_global_end"], cache["_local_end"] = info["current_end"], local_end
    slots, info, local_end = kvc.plan_cache_step(cache, 5 * blk, blk, blk, 5 * blk)
    assert info["action"] == "roll_and_insert"
    assert (info["num_evicted_tokens"], info["num_rolled_tokens"], info["sink_tokens"]) == (2640, 7920, 2640)
    assert (info["local_start_index"], local_end) == (10560, 13200)
    assert slots == (0, 2, 3, 4)  # sink slot, then the three surviving window slots
    cache["_global_end"], cache["_local_end"] = info["current_end"], local_end
    slots, info, local_end = kvc.plan_cache_step(cache, 5 * blk, blk, blk, 5 * blk)  # forwards 2..5 of that chunk
    assert info["action"] == "direct_insert" and slots == (0, 1, 2, 3) and info["local_start_index"] == 10560
    with pytest.raises(NotImplementedError):
        kvc.plan_cache_step(_fake_cache(blk, 5), 0, blk // 2, blk)


def test_nvfp4_checkpoint_helpers_on_plain_dictionaries():
    from types import SimpleNamespace

    from longlive_amd.utils import nvfp4_checkpoint as ck

    assert ck.is_nvfp4_state_dict({"blocks.0.ffn.0.quantized_weight_values": 1})
    assert not ck.is_nvfp4_state_dict({"blocks.0.ffn.0.weight": 1}) and not ck.is_nvfp4_state_dict(3)
    ckpt = {"generator": {"a": 1}, "generator_ema": {"a": 2}}
    assert ck.unwrap_generator_state_dict(ckpt) == {"a": 1}
    assert ck.unwrap_generator_state_dict(ckpt, use_ema=True) == {"a": 2}
    assert ck.unwrap_generator_state_dict({"model": {"b": 1}}) == {"b": 1}
    assert ck.unwrap_generator_state_dict({"c": 1}) == {"c": 1}
    assert ck.clean_fsdp_state_dict_keys({"m._fsdp_wrapped_module.w": 0}) == {"m.w": 0}
    assert ck.is_te_nvfp4_checkpoint({"checkpoint_format": "longlive_generator_te_nvfp4"})
    cfg = ck.build_model_quantization_config(SimpleNamespace(model_quant_scale_rule="mse"))
    assert cfg.scale_rule.value == "mse" and cfg.activation_scale_rule.value == "mse" and not cfg.keep_master_weights
    assert ck.build_model_quantization_config(None).scale_rule.value == "static_6"


# --------------------------------------------------------------------------- attention: division of a launch
def test_attention_plan_for_the_benchmark_shapes():
    """The launcher's choice, as pure host arithmetic.  configs[2] has 24 x 10 full tiles of 256 queries and 24
    tiles of 80 queries (three of eight waves busy: 11 sixteenths of the cost) on 256 CUs: the full tiles run whole
    on 240 workgroups and the other 16 share the light ones.  The released shape (27 full groups of queries and
    one of 128 per head) runs two whole rounds; whole left-over tiles would make that three, so the 136 full and
    24 light tiles behind the rounds are shared by all workgroups, by cost.  Cross-attention of the same 2640
    queries over 512 text keys takes the first shape too (two rounds of 128-query tiles cost more outside their
    four iterations than inside); with 880 queries one round of 128-query tiles is best, with 7040 three rounds
    of 256-query tiles.  A forced split with nothing to split falls back to whole tiles."""
    from helpers import attention_full_plan

    plan = _native.attention_plan
    assert plan(2640, 24, 13200) == {"division": "split", "workgroups": 256, "whole_rounds": 0, "split_tiles": 24}
    full = attention_full_plan(2640, 24, 13200)
    assert (full["extra"], full["full_units"], full["units"], full["light"], full["full_qtiles"]) == (240, 0, 24 * 104, 11, 10)
    assert plan(7040, 24, 28160) == {"division": "split", "workgroups": 256, "whole_rounds": 2, "split_tiles": 160}
    full = attention_full_plan(7040, 24, 28160)
    assert (full["extra"], full["full_units"], full["light"], full["full_qtiles"], full["n_qtiles"]) == (0, 136 * 220, 12, 27, 28)
    assert plan(2640, 24, 512) == {"division": "split", "workgroups": 256, "whole_rounds": 0, "split_tiles": 24}
    assert plan(880, 24, 512)["division"] == "narrow" and plan(880, 24, 512)["workgroups"] == 24 * 7
    assert plan(7040, 24, 512) == {"division": "wide", "workgroups": 672, "whole_rounds": 1, "split_tiles": 0}
    assert plan(2560, 24, 4096) == {"division": "wide", "workgroups": 240, "whole_rounds": 1, "split_tiles": 0}
    assert plan(2048, 32, 4096, policy="split")["division"] == "wide"   # 256 tiles: nothing is left to split
    assert plan(5, 1, 3000, policy="split") == {"division": "split", "workgroups": 13, "whole_rounds": 0, "split_tiles": 1}
    assert plan(2640, 24, 13200, compute_units=304)["division"] == "split"
    with pytest.raises(ValueError):
        plan(0, 24, 100)


def _check_division(plan, tiles):
    """Every (tile, iteration) in exactly one segment; whole tiles first; the parts of a split tile held by exactly
    the workgroups parts_of_tile names, one part each, in records no two parts share; at most two partial tiles
    per share; shares of equal cost to within one unit."""
    from helpers import DIVISION_FIELDS, attention_parts, attention_record, attention_segments

    d = {k: plan[k] for k in DIVISION_FIELDS}
    G, rounds, extra, n_iter = d["G"], d["whole_rounds"], d["extra"], d["n_iter"]
    assert rounds * G + extra + plan["split_tiles"] == tiles and d["units"] == plan["split_tiles"] * n_iter
    assert d["full_units"] <= d["units"] and d["full_units"] % n_iter == 0 and 9 <= d["light"] <= 16
    covered = np.zeros((tiles, n_iter), dtype=np.int32)
    holders, records, costs = {}, set(), []
    for g in range(G):
        segs = attention_segments(d, g)
        whole = rounds + (1 if g < extra else 0)
        assert [s[0] for s in segs[:whole]] == [j * G + g for j in range(whole)]
        assert all(s[1] == 0 and s[2] == n_iter for s in segs[:whole])
        assert g >= extra or len(segs) == whole          # a workgroup with an extra tile takes no share
        partial, cost = 0, 0
        for tile, begin, end in segs[whole:]:
            split_tile = tile - rounds * G - extra
            cost += (end - begin) * (16 if split_tile * n_iter < d["full_units"] else d["light"])
        for tile, begin, end in segs:
            assert 0 <= begin < end <= n_iter
            covered[tile, begin:end] += 1
            if (begin, end) != (0, n_iter):
                partial += 1
                split_tile = tile - rounds * G - extra
                holders.setdefault(split_tile, []).append(g)
                rec = attention_record(g, split_tile, d)
                assert rec in (2 * g, 2 * g + 1) and rec not in records
                records.add(rec)
        assert partial <= 2
        if g >= extra and d["units"]:
            assert cost > 0
            costs.append(cost)
    assert (covered == 1).all()
    if costs:
        assert max(costs) - min(costs) <= 2 * 16
    for split_tile, gs in holders.items():
        first, last = attention_parts(split_tile, d)
        assert gs == list(range(first, last + 1)), (split_tile, gs, first, last)


def test_attention_work_division_covers_every_iteration_exactly_once():
    """The kernel's own division arithmetic (csrc/attention_split.h, compiled for the host by the test-only
    library) for the launcher's plans of a spread of shapes - light last tiles, none, only light tiles, more and
    fewer tiles than compute units - and for hand-made divisions the launcher would not choose."""
    from helpers import attention_full_plan

    cases = [(2640, 24, 13200, 256), (7040, 24, 28160, 256), (300, 3, 1500, 256), (2000, 40, 200, 256),
             (5, 1, 3000, 256), (3000, 36, 700, 256), (1320, 24, 13200, 256), (2640, 24, 13200, 304),
             (2640, 24, 13200, 80), (777, 5, 999, 7), (2560, 30, 5000, 256), (100, 300, 640, 256),
             (2640, 24, 2640, 256), (2640, 24, 5280, 256), (2640, 24, 7920, 256), (2640, 24, 10560, 256),
             (64, 1, 14, 256), (1, 1, 1, 256), (200, 2, 100, 256), (129, 3, 128, 4)]
    rng = np.random.default_rng(11)
    cases += [(int(rng.integers(1, 9000)), int(rng.integers(1, 48)), int(rng.integers(1, 40000)), int(rng.choice([8, 64, 256, 304])))
              for _ in range(60)]
    split_seen = 0
    for Lq, H, n_keys, cus in cases:
        plan = attention_full_plan(Lq, H, n_keys, cus, policy=2)
        tiles = H * -(-Lq // 256)
        assert plan["n_iter"] == -(-n_keys // 128) and plan["n_qtiles"] == -(-Lq // 256)
        if plan["mode"] != 2:
            assert plan["G"] == tiles and plan["whole_rounds"] == 1 and plan["units"] == 0 and plan["extra"] == 0
            assert plan["full_qtiles"] == plan["n_qtiles"]
            continue
        split_seen += 1
        # the tile numbering: full groups of queries first, head by head, the light last groups behind them
        light_tiles = H if 1 <= Lq % 256 <= 128 else 0   # busy waves with a SIMD each
        assert plan["full_qtiles"] == plan["n_qtiles"] - (1 if light_tiles else 0)
        assert plan["units"] - plan["full_units"] == light_tiles * plan["n_iter"]
        _check_division(plan, tiles)
    assert split_seen > 40
    # hand-made divisions, the last two large enough to leave the 32-bit arithmetic
    for G, rounds, extra, full_split, light_split, light, n_iter in [
            (16, 0, 0, 20, 0, 16, 50), (16, 1, 5, 0, 7, 11, 50), (16, 2, 15, 3, 9, 9, 50), (7, 0, 3, 2, 2, 13, 50),
            (32, 0, 0, 0, 5, 10, 50), (8, 3, 0, 9, 1, 15, 50), (256, 0, 0, 3, 5, 11, 400000), (256, 1, 200, 2, 7, 12, 300001)]:
        plan = dict(mode=2, n_iter=n_iter, G=G, whole_rounds=rounds, extra=extra, units=(full_split + light_split) * n_iter,
                    full_units=full_split * n_iter, light=light, split_tiles=full_split + light_split)
        _check_division(plan, rounds * G + extra + full_split + light_split)


def test_persistent_gemm_division_covers_every_k_step_exactly_once():
    """The persistent GEMM's division of a launch between workgroups (longlive_amd/csrc/gemm_split.h, the functions
    the kernel calls, compiled for the host): over the launcher's plans for the benchmark shapes, the released
    shapes, grouped products and a sweep of random sizes and compute-unit counts, every (tile, K step) is computed
    exactly once, shares of the split part differ by at most one step, only the first and the last tile of a share
    are partial, every workgroup between the first and the last holder of a split tile holds a part of it, and no
    two parts that meet in one tile use the same record."""
    from helpers import GEMM_DIVISION_FIELDS, gemm_parts, gemm_plan, gemm_record, gemm_segments

    rng = np.random.default_rng(5)
    shapes = [(2640, 14336, 3072, 1, 256), (2640, 3072, 14336, 1, 256), (2640, 3072, 3072, 3, 256), (2640, 3072, 3072, 1, 256),
              (7040, 14336, 3072, 1, 256), (7040, 3072, 14336, 1, 256), (512, 3072, 3072, 2, 256), (128, 512, 128 * 300, 1, 256),
              (4096, 4096, 14336, 1, 256), (129, 513, 256, 4, 8), (2640, 3072, 14336, 1, 304), (300, 700, 1280, 1, 7)]
    for _ in range(30):
        shapes.append((int(rng.integers(1, 6000)), int(rng.integers(1, 9000)), 128 * int(rng.integers(1, 120)),
                       int(rng.integers(1, 5)), int(rng.choice([1, 8, 64, 104, 256, 304]))))
    used = 0
    for M, N, Kp, n_products, cus in shapes:
        plan = gemm_plan(M, N, Kp, n_products, cus)
        if not plan["use"]:
            assert plan["tiles"] == 0 or True
            continue
        used += 1
        d = {k: plan[k] for k in GEMM_DIVISION_FIELDS}
        G, tiles, nk, rounds = (d[k] for k in GEMM_DIVISION_FIELDS)
        assert G == cus and tiles == plan["tiles_m"] * plan["tiles_n_each"] * n_products and nk == Kp // 128
        assert plan["tiles_m"] * 128 >= M and plan["tiles_n_each"] * 512 >= N and rounds * G <= tiles
        covered = np.zeros((tiles, nk), dtype=np.int32)
        split = tiles - rounds * G
        holders = [set() for _ in range(split)]
        records = [dict() for _ in range(split)]
        share_sizes = []
        for g in range(G):
            segs = gemm_segments(d, g)
            assert [t for t, _, _ in segs[:rounds]] == [j * G + g for j in range(rounds)]
            steps = 0
            partial = []
            for i, (t, b, e) in enumerate(segs):
                assert 0 <= t < tiles and 0 <= b < e <= nk, (M, N, Kp, g, t, b, e)
                covered[t, b:e] += 1
                if i >= rounds:
                    steps += e - b
                    st = t - rounds * G
                    holders[st].add(g)
                    if b != 0 or e != nk:
                        partial.append(i)
                        rec = gemm_record(g, st, d)
                        assert rec // 2 == g and rec not in records[st].values()
                        records[st][g] = rec
            share_sizes.append(steps)
            assert all(i in (rounds, len(segs) - 1) for i in partial)            # first walked = last tile of the share, and vice versa
            assert len({gemm_record(g, segs[i][0] - rounds * G, d) for i in partial}) == len(partial)   # its two parts: two records
        assert (covered == 1).all(), (M, N, Kp, n_products, cus)
        if split:
            assert max(share_sizes) - min(share_sizes) <= 1 and min(share_sizes) >= 1
        for st in range(split):
            first, last = gemm_parts(st, d)
            assert holders[st] == set(range(first, last + 1)), (M, N, Kp, st, first, last, holders[st])
    assert used >= 20


def test_persistent_gemm_plan_for_the_benchmark_shapes():
    """The launcher's choice for the shapes of the benchmark on 256 compute units: the automatic choice runs one
    workgroup per tile everywhere (the persistent launch measured slower inside the block); on request, FFN-down
    runs as 126 tiles of 112 K steps, each shared by two workgroups; a K that is not a multiple of 128, or less work
    than one K step per workgroup, never runs persistently."""
    from longlive_amd import _native

    assert not _native.gemm_plan(2640, 3072, 14336)["persistent"]
    assert not _native.gemm_plan(2640, 14336, 3072)["persistent"]
    down = _native.gemm_plan(2640, 3072, 14336, schedule="persistent")
    assert down == {"persistent": True, "workgroups": 256, "tiles": 126, "k_steps": 112}
    assert _native.gemm_plan(2640, 14336, 3072, schedule="persistent")["persistent"]
    assert _native.gemm_plan(512, 3072, 3072, n_products=2, schedule="persistent")["persistent"]
    assert not _native.gemm_plan(2640, 3072, 14336, schedule="tiles")["persistent"]
    assert not _native.gemm_plan(2640, 3072, 14336 + 64, schedule="persistent")["persistent"]
    assert not _native.gemm_plan(64, 64, 128, schedule="persistent")["persistent"]


def test_generated_gemm_loops_in_the_tree_are_what_their_generators_write(tmp_path):
    """The hand-scheduled main loops are generated text kept in the tree; a generator edited without regenerating
    (or a generated file edited by hand) would build a library that no longer matches its source."""
    import os
    import subprocess
    import sys
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "longlive_amd", "csrc")
    cases = [("gemm_loop_gfx950.inc", ["gemm_loop_gen.py", "{out}"]),
             ("gemm_tile_loop_42_gfx950.inc", ["gemm_tile_loop_gen.py", "4", "2", "{out}"]),
             ("gemm_tile_loop_24_gfx950.inc", ["gemm_tile_loop_gen.py", "2", "4", "{out}"]),
             ("gemm_tile_loop_24w8_gfx950.inc", ["gemm_tile_loop_gen.py", "2", "4", "{out}", "--waves", "8"])]
    for name, cmd in cases:
        out = str(tmp_path / name)
        subprocess.run([sys.executable, os.path.join(csrc, cmd[0])] + [a.format(out=out) for a in cmd[1:]], check=True, cwd=csrc)
        with open(out) as got, open(os.path.join(csrc, name)) as kept:
            assert got.read() == kept.read(), name


def test_which_gemm_kernel_the_shapes_of_the_block_take():
    """ll_nvfp4_gemm_kernel (host arithmetic): on 256 compute units FFN-up takes the 256 x 128 tile and the grouped
    q / k / v launch the 128 x 256 tile, both with the hand-scheduled loop; the 2640 x 3072 products take the
    eight-wave kernel; the M = 512 text projections 64 x 64 tiles; a K that is not a multiple of 128, or the schedule
    that asks for it, the compiled loops; the persistent schedule only when asked for."""
    k = _native.gemm_kernel
    assert k(2640, 14336, 3072) == {"kernel": "256x128", "hand_scheduled": True}
    assert k(2640, 3072, 3072, n_products=3) == {"kernel": "128x256", "hand_scheduled": True}
    for K in (3072, 14336):
        assert k(2640, 3072, K) == {"kernel": "eight_waves", "hand_scheduled": True}
    assert k(1760, 3072, 3072)["kernel"] == "eight_waves" and k(880, 3072, 3072, n_products=3)["kernel"] == "eight_waves"
    assert k(880, 3072, 3072)["kernel"] != "eight_waves"          # 84 tiles: less than half of the units
    assert k(7040, 3072, 3072)["kernel"] == "256x128"             # 660 tiles of 128 x 256: more than one per unit
    assert k(512, 3072, 3072) == {"kernel": "64x64", "hand_scheduled": False}
    assert k(2640, 3072, 3072 + 64) == {"kernel": "128x128", "hand_scheduled": False}
    assert k(2640, 3072, 384)["kernel"] == "128x128"              # fewer than four K steps
    assert k(2640, 3072, 3072, schedule="tiles_compiled") == {"kernel": "128x128", "hand_scheduled": False}
    assert k(2640, 14336, 3072, schedule="tiles_compiled") == {"kernel": "256x128", "hand_scheduled": False}
    assert k(2640, 14336, 3072, schedule="persistent") == {"kernel": "persistent", "hand_scheduled": True}
    assert k(2640, 3072, 3072, compute_units=128)["kernel"] != "eight_waves"   # 252 tiles on 128 units
    with pytest.raises(Exception):
        k(0, 3072, 3072)
