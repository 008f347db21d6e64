"""Shared helpers of the test-suite: bf16 bit views and the benchmark input distributions."""
import numpy as np
import torch

from longlive_amd.utils.synthetic import activations, bits_of, u8, weights  # noqa: F401  (shared with bench.py and the smoke test)


def from_bits(b: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16).to(device)


def f32_of(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def hardware_convert(x: torch.Tensor, mode: int) -> torch.Tensor:
    """fp32 -> e4m3 byte (mode 0) or e2m1 nibble (mode 1) with the gfx950 conversion instructions, through the
    test-only library built next to the product library (longlive_amd/csrc/test_hooks.hip)."""
    import ctypes
    import os

    from longlive_amd import _native

    path = os.path.join(os.path.dirname(_native.LIB_PATH), "libll_nvfp4_testhooks.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `make -C longlive_amd/csrc`")
    lib = ctypes.CDLL(path)
    lib.ll_test_convert.restype = ctypes.c_int
    lib.ll_test_convert.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    x = x.contiguous().float()
    out = torch.empty(x.numel(), dtype=torch.uint8, device=x.device)
    code = lib.ll_test_convert(x.data_ptr(), x.numel(), mode, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    if code != 0:
        raise RuntimeError(f"ll_test_convert failed with {code}")
    return out


def block_oracle_params(block) -> dict:
    """Parameters of a (quantized) DiTBlock in the form oracle/dit_oracle.block_forward takes."""
    f = lambda t: t.detach().float().cpu().numpy()
    p = {"modulation": f(block.modulation)[0]}
    for name in ("self_attn.q", "self_attn.k", "self_attn.v", "self_attn.o", "cross_attn.q", "cross_attn.k",
                 "cross_attn.v", "cross_attn.o", "ffn.0", "ffn.2"):
        lin = block.get_submodule(name)
        qw = lin.quantized_weight()
        p[name + ".w"] = dict(values=u8(qw.values), scales=u8(qw.scale_factors), amax=np.float32(qw.amax.item()),
                              rule=qw.scale_rule.value, padded=tuple(qw.padded_shape), orig=tuple(qw.original_shape))
        p[name + ".b"] = f(lin.bias)
    for name in ("self_attn.norm_q", "self_attn.norm_k", "cross_attn.norm_q", "cross_attn.norm_k"):
        p[name] = f(block.get_submodule(name).weight)
    p["norm3.w"], p["norm3.b"] = f(block.norm3.weight), f(block.norm3.bias)
    return p


def generator_oracle_params(model) -> dict:
    """Parameters of a quantized CausalDiT in the form oracle/generator_oracle takes: bf16 CPU tensors for the
    embeddings and the head, block_oracle_params per block."""
    c = lambda t: t.detach().cpu().bfloat16()
    P = {"patch_embedding.weight": c(model.patch_embedding.weight), "patch_embedding.bias": c(model.patch_embedding.bias),
         "head.modulation": c(model.head.modulation), "head.head.weight": c(model.head.head.weight),
         "head.head.bias": c(model.head.head.bias)}
    for name, seq, idx in (("time_embedding", model.time_embedding, (0, 2)), ("text_embedding", model.text_embedding, (0, 2)),
                           ("time_projection", model.time_projection, (1,))):
        for i in idx:
            P[f"{name}.{i}.weight"], P[f"{name}.{i}.bias"] = c(seq[i].weight), c(seq[i].bias)
    P["blocks"] = [block_oracle_params(b) for b in model.blocks]
    return P


def _test_hooks():
    import ctypes
    import os

    from longlive_amd import _native

    path = os.path.join(os.path.dirname(_native.LIB_PATH), "libll_nvfp4_testhooks.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `make -C longlive_amd/csrc`")
    return ctypes.CDLL(path)


DIVISION_FIELDS = ("G", "whole_rounds", "extra", "n_iter", "units", "full_units", "light")


def _division_array(division: dict):
    import ctypes

    return (ctypes.c_uint32 * 7)(*[int(division[k]) for k in DIVISION_FIELDS])


def attention_segments(division: dict, g: int):
    """The (tile, begin, end) segments workgroup g walks, in order, from the attention kernel's own division
    arithmetic compiled for the host (longlive_amd/csrc/attention_split.h through the test-only library).
    ``division`` has the keys of DIVISION_FIELDS."""
    import ctypes

    lib = _test_hooks()
    lib.ll_test_attention_segments.restype = ctypes.c_int
    lib.ll_test_attention_segments.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int]
    buf = (ctypes.c_int32 * (3 * 4096))()
    n = lib.ll_test_attention_segments(_division_array(division), g, buf, 4096)
    assert n <= 4096
    return [(buf[3 * i], buf[3 * i + 1], buf[3 * i + 2]) for i in range(n)]


def attention_parts(split_tile: int, division: dict):
    import ctypes

    lib = _test_hooks()
    lib.ll_test_attention_parts.restype = None
    lib.ll_test_attention_parts.argtypes = [ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    first, last = ctypes.c_uint32(), ctypes.c_uint32()
    lib.ll_test_attention_parts(split_tile, _division_array(division), ctypes.byref(first), ctypes.byref(last))
    return first.value, last.value


def attention_record(g: int, split_tile: int, division: dict) -> int:
    import ctypes

    lib = _test_hooks()
    lib.ll_test_attention_record.restype = ctypes.c_uint32
    lib.ll_test_attention_record.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p]
    return lib.ll_test_attention_record(g, split_tile, _division_array(division))


def attention_full_plan(Lq: int, H: int, n_keys: int, cus: int = 256, policy: int = -1) -> dict:
    """The launcher's choice for a shape, division included: mode (0 narrow, 1 wide, 2 split), n_qtiles,
    full_qtiles, split_tiles and the keys of DIVISION_FIELDS."""
    import ctypes

    lib = _test_hooks()
    lib.ll_test_attention_full_plan.restype = None
    lib.ll_test_attention_full_plan.argtypes = [ctypes.c_int64, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                                ctypes.c_void_p]
    out = (ctypes.c_uint32 * 11)()
    lib.ll_test_attention_full_plan(Lq, H, n_keys, cus, policy, out)
    plan = dict(mode=out[0], n_qtiles=out[1], full_qtiles=out[2], split_tiles=out[3])
    plan.update({k: out[4 + i] for i, k in enumerate(DIVISION_FIELDS)})
    return plan


def attention_division_on_device(division: dict, split_tiles: int, device):
    """first_unit_of(g) for g = 0 .. G and (first, last) holder of every split tile, computed by a kernel that calls the
    same functions as the attention kernel; and the host's values for the same division."""
    import ctypes

    import torch

    lib = _test_hooks()
    lib.ll_test_attention_division_on_device.restype = ctypes.c_int
    lib.ll_test_attention_division_on_device.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p]
    lib.ll_test_attention_first_unit.restype = ctypes.c_uint32
    lib.ll_test_attention_first_unit.argtypes = [ctypes.c_uint32, ctypes.c_void_p]
    arr = _division_array(division)
    G = int(division["G"])
    out = torch.zeros(G + 1 + 2 * split_tiles, dtype=torch.int32, device=device)
    rc = lib.ll_test_attention_division_on_device(arr, split_tiles, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.uint32)
    host = [lib.ll_test_attention_first_unit(g, arr) for g in range(G + 1)]
    host += [x for t in range(split_tiles) for x in attention_parts(t, division)]
    return got, np.array(host, dtype=np.uint32)


GEMM_DIVISION_FIELDS = ("G", "tiles", "nk", "whole_rounds")


def gemm_plan(M: int, N: int, Kp: int, n_products: int = 1, cus: int = 256, schedule: int = 1) -> dict:
    """The GEMM launcher's choice for a shape from the same arithmetic compiled for the host
    (longlive_amd/csrc/gemm_split.h): use (persistent launch or not), the keys of GEMM_DIVISION_FIELDS, tiles_m and
    tiles_n_each.  schedule: -1 automatic, 0 one workgroup per tile, 1 persistent wherever possible."""
    import ctypes

    lib = _test_hooks()
    lib.ll_test_gemm_plan.restype = None
    lib.ll_test_gemm_plan.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_void_p]
    out = (ctypes.c_uint32 * 7)()
    lib.ll_test_gemm_plan(M, N, Kp, n_products, cus, schedule, out)
    return dict(use=bool(out[0]), G=out[1], tiles=out[2], nk=out[3], whole_rounds=out[4], tiles_m=out[5], tiles_n_each=out[6])


def gemm_segments(division: dict, g: int):
    """The (tile, begin, end) segments workgroup g of the persistent GEMM walks, in order."""
    import ctypes

    lib = _test_hooks()
    lib.ll_test_gemm_segments.restype = ctypes.c_int
    lib.ll_test_gemm_segments.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int]
    arr = (ctypes.c_uint32 * 4)(*[int(division[k]) for k in GEMM_DIVISION_FIELDS])
    buf = (ctypes.c_int32 * (3 * 4096))()
    n = lib.ll_test_gemm_segments(arr, g, buf, 4096)
    assert n <= 4096
    return [(buf[3 * i], buf[3 * i + 1], buf[3 * i + 2]) for i in range(n)]


def gemm_parts(split_tile: int, division: dict):
    import ctypes

    lib = _test_hooks()
    lib.ll_test_gemm_parts.restype = None
    lib.ll_test_gemm_parts.argtypes = [ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    arr = (ctypes.c_uint32 * 4)(*[int(division[k]) for k in GEMM_DIVISION_FIELDS])
    first, last = ctypes.c_uint32(), ctypes.c_uint32()
    lib.ll_test_gemm_parts(split_tile, arr, ctypes.byref(first), ctypes.byref(last))
    return first.value, last.value


def gemm_record(g: int, split_tile: int, division: dict) -> int:
    import ctypes

    lib = _test_hooks()
    lib.ll_test_gemm_record.restype = ctypes.c_uint32
    lib.ll_test_gemm_record.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p]
    arr = (ctypes.c_uint32 * 4)(*[int(division[k]) for k in GEMM_DIVISION_FIELDS])
    return lib.ll_test_gemm_record(g, split_tile, arr)
