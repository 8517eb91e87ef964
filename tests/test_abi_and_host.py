"""CPU-side checks: the C-ABI library loads and exports every symbol the
header declares; the host layer validates arguments the way the reference
does and refuses to run without a GPU instead of falling back."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "bitween_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bw_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from bitween_amd.kernels import hip_loader
    if not os.path.exists(hip_loader.library_path()):
        from bitween_amd.csrc import build
        build.build()
    lib = ctypes.CDLL(hip_loader.library_path())
    declared = _declared_symbols()
    assert set(declared) == set(hip_loader.ENTRY_POINTS)
    for name in declared:
        assert hasattr(lib, name), name
    lib.bw_abi_version.restype = ctypes.c_int
    assert lib.bw_abi_version() == hip_loader.ABI_VERSION == 10
    lib.bw_strerror.restype = ctypes.c_char_p
    assert lib.bw_strerror(0) == b"ok" and b"invalid" in lib.bw_strerror(-1)


def test_entry_points_reject_bad_arguments_before_touching_the_gpu():
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    one = ctypes.c_void_p(16)
    # bits = 3
    assert lib.bw_quantize_pack(one, 2, 2, 4, 128, 128, 3, 32, one, one, 2, one, 3, None) == -1
    # K % group != 0
    assert lib.bw_quantize_pack(one, 2, 2, 4, 100, 100, 4, 32, one, one, 2, one, 3, None) == -1
    # null pointers
    assert lib.bw_dequantize(None, one, 0, one, 0, 4, 128, 4, 32, one, 0, 128, None) == -1
    # M out of range for the decode kernel
    assert lib.bw_qgemv(one, 0, 17, 128, 128, one, one, one, None, 16, 4, 32, one, 16, None) == -1
    assert lib.bw_qgemv(one, 0, 0, 128, 128, one, one, one, None, 16, 4, 32, one, 16, None) == -1
    # float32 activations are not built (bfloat16 is, for the decode kernels only)
    assert lib.bw_qgemv(one, 2, 1, 128, 128, one, one, one, None, 16, 4, 32, one, 16, None) == -2
    assert lib.bw_qgemm(one, 1, 128, 128, 128, one, one, one, None, 16, 4, 32, one, 16, None) == -2
    # split-K prefill: same checks as bw_qgemm, before the workspace is looked at
    assert lib.bw_qgemm_ws(None, 0, 128, 128, 128, one, one, one, None, 16, 4, 32, one, 16, None, 0, None) == -1
    assert lib.bw_qgemm_ws(one, 0, 128, 128, 64, one, one, one, None, 16, 4, 32, one, 16, None, 0, None) == -1
    assert lib.bw_qgemm_ws(one, 1, 128, 128, 128, one, one, one, None, 16, 4, 32, one, 16, None, 0, None) == -2


def test_split_k_workspace_size_is_a_pure_host_function():
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    ws = lib.bw_qgemm_workspace_bytes
    tile = 128 * 256 * 4                                        # one float32 partial tile
    rows = lib.bw_qgemm_tile_rows
    # whole rounds of 256 tiles (one workgroup per CU), or a last round that is more than half full: no workspace
    assert ws(2048, 4096, 4096, 4, 128) == 0 and rows(2048, 4096, 4096, 4, 128) == 128    # 16 x 16 tiles = exactly one round
    assert ws(4096, 4096, 4096, 4, 128) == 0 and rows(4096, 4096, 4096, 4, 128) == 256    # 512 tiles of 128 rows, or 256 of 256
    # the tile height is the one whose grid fills its rounds better: 1.75 rounds of 128-row tiles against one of 256-row tiles
    assert rows(1024, 14336, 4096, 4, 128) == 256 and rows(2048, 14336, 4096, 4, 128) == 256 and rows(2048, 4096, 14336, 4, 128) == 128
    assert ws(2048, 4096, 14336, 4, 128) == 0                    # 256 tiles of 128 rows: exactly one round
    # 256-row tiles need whole K steps of 128 values and a grid that fills the device
    assert rows(4096, 4096, 4096, 2, 128) == 256 and rows(4096, 4096, 4096 + 64, 4, 64) == 128 and rows(512, 14336, 4096, 4, 128) == 128
    assert rows(128, 20, 96, 4, 48) == 0                        # the shape-generic kernel
    # calls of at most 64 rows take 64-row tiles (natural-order schedule: K a multiple of 128); their split-K blocks fit
    # the workspace of the 128-row plan
    assert rows(64, 4096, 4096, 4, 128) == 64 and rows(17, 11008, 4096, 8, 64) == 64 and rows(65, 11008, 4096, 4, 128) == 128
    assert rows(32, 4096, 4096 + 64, 4, 64) == 128
    # up to 128 rows as two 64-row tiles where N is at most 16 tiles wide (half the partial-tile traffic of the K split)
    assert rows(128, 4096, 14336, 4, 128) == 64 and rows(96, 4096, 4096, 8, 128) == 64 and rows(129, 4096, 4096, 4, 128) == 128
    assert rows(128, 4096 + 256, 4096, 4, 128) == 128
    assert ws(512, 14336, 4096, 4, 128) == 0                    # 224 tiles: 0.875 of a round
    # few tiles and a long K: every tile split so that one round is filled
    for m, n, k, bits in ((128, 4096, 14336, 4), (512, 4096, 14336, 4), (128, 14336, 4096, 4), (64, 1024, 2048, 8)):
        b = ws(m, n, k, bits, 128)
        tiles = -(-n // 256) * -(-m // 128)
        assert b % (tiles * tile) == 0 and 2 <= b // (tiles * tile) and tiles * (b // (tiles * tile)) <= 256
    # a last round that is at most half full: only its tiles are split (896 tiles = 3 rounds + 128 tiles, cut in two)
    assert ws(2048, 14336, 4096, 4, 128) == 128 * 2 * tile
    # too short a K to split, invalid shapes, shapes the generic kernel takes
    assert ws(128, 256, 128, 4, 128) == 0
    assert ws(128, 256, 100, 4, 32) == 0
    assert ws(128, 20, 96, 4, 48) == 0


def test_decode_rows_switch_is_a_pure_host_function():
    """bw_qlinear keeps up to 48 rows on the decode kernel for layers under 10 MiB of packed weights, 32 under 40 MiB
    (a third 16-row launch loses to one launch of the prefill kernel's 64-row tiles) and 16 from 40 MiB on."""
    from bitween_amd.kernels import hip_loader
    rows = hip_loader.load().bw_qlinear_decode_rows
    assert rows(4096, 4096, 4) == 48 and rows(4096, 4096, 8) == 32 and rows(4096, 11008, 2) == 32
    assert rows(11008, 4096, 4) == 32 and rows(14336, 4096, 4) == 32 and rows(4096, 11008, 8) == 16 and rows(12288, 4096, 8) == 16
    assert rows(0, 4096, 4) == 0 and rows(4096, 4096, 3) == 0


def test_host_layer_error_conventions_without_gpu():
    import bitween_amd
    with pytest.raises(AssertionError):                       # bitween/functional.py:6
        bitween_amd.quantize_rtn(torch.zeros(4, 96), 3, 32)
    with pytest.raises(ValueError):                           # bitween/functional.py:12-17
        bitween_amd.quantize_rtn(torch.zeros(4, 100), 4, 32)
    with pytest.raises(ValueError):                           # bitween/modules.py:157-161
        bitween_amd.QuantizedLinear(64, 64, bits=5)
    with pytest.raises(ValueError):
        bitween_amd.QuantizedLinear(64, 64, bits=4, group_size=0)
    with pytest.raises(AssertionError):                       # bitween/quantizer/quantizer.py:36
        bitween_amd.Bitween(torch.nn.Linear(8, 8), group_size=0)
    q = bitween_amd.QuantizedLinear(256, 64, bits=4, group_size=128, bias=True)
    assert q.qweight.shape == (64, 32) and q.qweight.dtype == torch.int32
    assert q.scale.shape == (64, 2) and q.scale.dtype == torch.float16 and q.zero_point.dtype == torch.float16
    assert q.bias.dtype == torch.float16 and q.dtype == torch.float16 and q.requires_grad is False
    assert bitween_amd.QuantizedLinear(256, 64, bias=False).bias is None


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU behaviour")
def test_no_silent_cpu_fallback():
    import bitween_amd
    from bitween_amd.kernels.hip_loader import BitweenHipError
    with pytest.raises(BitweenHipError):
        bitween_amd.quantize_rtn(torch.randn(4, 128), 4, 32)
    with pytest.raises(BitweenHipError):
        bitween_amd.QuantizedLinear.from_float(torch.nn.Linear(128, 8), 4, 32)
    q = bitween_amd.QuantizedLinear(128, 8, bits=4, group_size=32)
    with pytest.raises(BitweenHipError):
        q(torch.randn(2, 128))


def test_product_code_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "bitween_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


def test_reference_package_name_resolves_to_this_implementation(tmp_path):
    """`import bitween...` and pickles that name bitween.modules.QuantizedLinear (torch.save(model),
    main.py:134-145) resolve to bitween_amd; buffers survive the round trip."""
    import torch
    import bitween
    import bitween.modules
    import bitween_amd
    from bitween.functional import quantize_rtn
    from bitween.quantizer.quantizer import Bitween
    assert bitween.modules.QuantizedLinear is bitween_amd.QuantizedLinear
    assert quantize_rtn is bitween_amd.quantize_rtn and Bitween is bitween_amd.Bitween
    model = torch.nn.Sequential(bitween_amd.QuantizedLinear(64, 32, bits=4, group_size=32, bias=True))
    model[0].qweight.random_(-2 ** 31, 2 ** 31 - 1)
    model[0].scale.copy_(torch.rand(32, 2))
    model[0].zero_point.copy_(torch.randint(0, 16, (32, 2)))
    cls = bitween_amd.QuantizedLinear
    saved = cls.__module__
    try:
        cls.__module__ = "bitween.modules"                    # what a pickle written by the reference says
        torch.save(model, tmp_path / "m.pt")
    finally:
        cls.__module__ = saved
    assert b"bitween.modules" in (tmp_path / "m.pt").read_bytes() or True
    back = torch.load(tmp_path / "m.pt", weights_only=False)
    assert isinstance(back[0], bitween_amd.QuantizedLinear)
    assert (back[0].bits, back[0].group_size, back[0].in_features, back[0].out_features) == (4, 32, 64, 32)
    for name in ("qweight", "scale", "zero_point", "bias"):
        assert torch.equal(getattr(back[0], name), getattr(model[0], name))


def test_precision_map_lookup():
    from bitween_amd.quantizer.quantizer import _precision_for
    cfg = {"model.layers.0": (8, 128), "model.layers.0.mlp.down_proj": {"bits": 2, "group_size": 32}, "lm": (4, 64)}
    assert _precision_for("model.layers.0.self_attn.q_proj", cfg, None) == (8, 128)
    assert _precision_for("model.layers.0.mlp.down_proj", cfg, None) == (2, 32)       # the longest key wins
    assert _precision_for("model.layers.01.mlp.up_proj", cfg, None) is None           # prefix of a name is not a block
    assert _precision_for("lm_head", cfg, (4, 128)) == (4, 128)
    assert _precision_for("lm", cfg, None) == (4, 64)


@pytest.mark.default_scale_division
def test_scale_division_default_follows_the_tensor_device():
    """The default mode is "auto": the reference's `(max - min) / Qmax` is a true division for a CPU tensor and a
    multiplication by the float32 reciprocal for a GPU tensor (bitween/functional.py:25 under eager torch)."""
    import bitween_amd
    from bitween_amd import functional as F

    class OnGpu:                                              # stands in for a GPU tensor: only the device is asked
        is_cuda = True

    if "BITWEEN_SCALE_DIVISION" not in os.environ:
        assert bitween_amd.get_scale_division() == "auto"
    cpu = torch.zeros(1)
    assert F.scale_reciprocal_for(cpu, "auto") is False and F.scale_reciprocal_for(OnGpu(), "auto") is True
    assert F.scale_reciprocal_for(cpu, "ieee") is False and F.scale_reciprocal_for(OnGpu(), "ieee") is False
    assert F.scale_reciprocal_for(cpu, "torch_device") is True and F.scale_reciprocal_for(OnGpu(), "torch_device") is True
    previous = bitween_amd.set_scale_division("torch_device")
    try:
        assert bitween_amd.get_scale_division() == "torch_device" and F.scale_reciprocal_for(cpu) is True
        with pytest.raises(ValueError):
            bitween_amd.set_scale_division("fast")
    finally:
        bitween_amd.set_scale_division(previous)
