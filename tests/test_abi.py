"""The C-ABI library loads on a CPU-only host, exports every symbol include/qwhip.h declares, and its
host-side checks (size law, view validation, kernel-name table, error strings) behave as the
reference's operator API does.  No compute call is made here."""
import ctypes as C
import pathlib
import re

import pytest

from qwegn_amd import qwhip

ROOT = pathlib.Path(__file__).resolve().parent.parent


def _declared():
    text = (ROOT / "include" / "qwhip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qwhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(str(qwhip.LIB_PATH))
    names = _declared()
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/qwhip.h but not exported"
    assert sorted(qwhip.SIGNATURES) == names, "python binding and header disagree"


def test_block_size_law():
    """4 + group*bits/8 bytes for every supported pair, nothing else (QWAQBlock.swift:17-86)."""
    lib = qwhip.load()
    assert lib.qwhip_block_bytes(qwhip.KIND_HQ4_G32_M5, 4, 32) == 20
    assert lib.qwhip_block_bytes(qwhip.KIND_HQ4_G32_M5, 4, 64) == 0
    for kind in (qwhip.KIND_ROTATED_HQ, qwhip.KIND_NATIVE_AFFINE):
        for bits in (2, 3, 4, 6, 8):
            for group in (32, 64, 128, 256):
                assert lib.qwhip_block_bytes(kind, bits, group) == 4 + group * bits // 8
        assert lib.qwhip_block_bytes(kind, 5, 32) == 0
        assert lib.qwhip_block_bytes(kind, 4, 48) == 0
    assert lib.qwhip_block_bytes(7, 4, 32) == 0
    # the configurations' sizes: HQ8_G32 and HQ4_G64 are both 36 bytes
    assert lib.qwhip_block_bytes(qwhip.KIND_ROTATED_HQ, 8, 32) == 36 == lib.qwhip_block_bytes(qwhip.KIND_ROTATED_HQ, 4, 64)


def test_weight_view_validation_mirrors_failable_init():
    """QWWeightView.init? fails unless n > 0, k > 0, k % group == 0, the pair is supported and the bytes fit
    (QWWeightView.swift:107-118)."""
    lib = qwhip.load()
    buf = (C.c_uint8 * 4096)()
    base = C.addressof(buf)

    def v(n, k, kind, bits, group, nbytes=4096, ptr=base):
        view = qwhip.WeightView(ptr, nbytes, n, k, kind, bits, group)
        return lib.qwhip_weight_view_validate(C.byref(view))

    assert v(8, 64, qwhip.KIND_HQ4_G32_M5, 4, 32) == qwhip.OK
    assert v(8, 64, qwhip.KIND_HQ4_G32_M5, 4, 32, nbytes=8 * 2 * 20) == qwhip.OK
    assert v(8, 64, qwhip.KIND_HQ4_G32_M5, 4, 32, nbytes=8 * 2 * 20 - 1) == qwhip.E_BAD_WEIGHTS
    assert b"bytes" in lib.qwhip_last_error()
    assert v(0, 64, qwhip.KIND_HQ4_G32_M5, 4, 32) == qwhip.E_BAD_WEIGHTS
    assert v(8, 48, qwhip.KIND_HQ4_G32_M5, 4, 32) == qwhip.E_BAD_WEIGHTS
    assert v(8, 64, qwhip.KIND_ROTATED_HQ, 4, 64) == qwhip.OK
    assert v(8, 96, qwhip.KIND_ROTATED_HQ, 4, 64) == qwhip.E_BAD_WEIGHTS        # k % group
    assert v(8, 64, qwhip.KIND_ROTATED_HQ, 5, 32) == qwhip.E_BAD_WEIGHTS        # unsupported pair
    assert v(8, 64, qwhip.KIND_NATIVE_AFFINE, 8, 32) == qwhip.OK
    assert v(8, 64, qwhip.KIND_HQ4_G32_M5, 4, 32, ptr=None) == qwhip.E_NULL
    assert v(8, 64, qwhip.KIND_HQ4_G32_M5, 4, 32, ptr=base + 2) == qwhip.E_BAD_WEIGHTS
    assert lib.qwhip_weight_view_validate(None) == qwhip.E_NULL


def test_kernel_lookup_keys_are_the_reference_kernel_names():
    """hal.pipeline(name) succeeds for the kernels of the path and throws kernelMissing otherwise
    (QWHal.swift:291-322)."""
    lib = qwhip.load()
    launcher = C.c_char_p()
    table = {
        b"qwg_gemv_q4g_dx_h16_t4": b"qwhip_gemv", b"qwg_gemv_q4g_v4": b"qwhip_gemv", b"qwg_skinny_m3": b"qwhip_gemv",
        b"qwg_gemv_aq8_g32_v4": b"qwhip_gemv", b"qwg_gemv_aq4_g64_dx_h16_t4": b"qwhip_gemv",
        b"qwg_gemv_q4g_f32_v4": b"qwhip_gemv_f32", b"qwg_gemm_q4g_f32_bm32": b"qwhip_gemv_f32", b"qwg_gemv_aq8_g64_f32_v4": b"qwhip_gemv_f32",
        b"qwg_gemm_aq4_g32_f32_bm": b"qwhip_gemv_f32", b"qwg_gemv_aq3_g32_f32_v4_am": b"qwhip_head_argmax", b"qwg_h32_f32": b"qwhip_h32_f32",
        b"qwg_gemv_aq3_g32_v4": b"qwhip_gemv", b"qwg_gemv_aq6_g128_dx_h16_t4": b"qwhip_gemv", b"qwg_gemv_aq2_g64_v4": b"qwhip_gemv", b"qwg_gemm_aq3_g32_h16": b"qwhip_gemm", b"qwg_gemv_aq6_g64_silu_pair_dx_h16": b"qwhip_gemv_silu_pair",
        b"qwg_moe_nax_gemm_aq2_g128": b"qwhip_moe_grouped_gemm", b"qwg_moe_gateup_aq3_g32_f32_r1": b"qwhip_moe_gateup_decode",
        b"qwg_embed_aq_f32": b"qwhip_embed_aq_f32", b"qwg_silu_mul_f32": b"qwhip_silu_mul_f32", b"qwg_add_f32": b"qwhip_add_f32",
        b"qwg_moe_bridge_f16_to_f32": b"qwhip_moe_bridge_f16_to_f32", b"qwg_latent_norm_h32_f32": b"qwhip_latent_norm_h32_f32",
        b"qwg_gemv_q4g_silu_pair_dx_h16": b"qwhip_gemv_silu_pair", b"qwg_gemv_aq4_g32_silu_pair_dx_h16": b"qwhip_gemv_silu_pair",
        b"qwg_gemm_q4g_h16_swiglu": b"qwhip_gemm_swiglu", b"qwg_gemm_aq4_g64_h16_swiglu": b"qwhip_gemm_swiglu",
        b"qwg_gemm_q4g_h16": b"qwhip_gemm", b"qwg_gemm_aq8_g32_h16": b"qwhip_gemm", b"qwg_gemm_aq4_g64_nax_f32": b"qwhip_gemm",
        b"qwg_moe_route": b"qwhip_moe_route", b"qwg_moe_group_pairs_f32": b"qwhip_moe_group_pairs",
        b"qwg_moe_nax_gemm": b"qwhip_moe_grouped_gemm", b"qwg_moe_nax_split_f32_aq4_g64": b"qwhip_moe_grouped_gemm",
        b"qwg_moe_nax_split_aq4_g64_f32": b"qwhip_moe_grouped_gemm", b"qwg_head_gemv_aq4_g32_argmax": b"qwhip_head_argmax",
        b"qwg_moe_down_reduce_combine_f32": b"qwhip_moe_combine", b"qwg_moe_gateup_q4g_f32_r1": b"qwhip_moe_gateup_decode",
        b"qwg_moe_down_shared_combine_q4g_f32": b"qwhip_moe_down_decode", b"qwg_fwht32_f16": b"qwhip_fwht32",
        b"qwg_quantize_bf16_to_hq4_g32_m5": b"qwhip_quantize_hq4_g32",
        b"qwg_rmsnorm": b"qwhip_rmsnorm", b"qwg_rmsnorm_residual": b"qwhip_rmsnorm",
        b"qwg_head_gemv_q4g_argmax": b"qwhip_head_argmax", b"qwg_gemv_q4g_f32_v4_am": b"qwhip_head_argmax",
        b"qwg_repack_mlx_affine_to_aq_m5": b"qwhip_repack_mlx_affine",
        b"qwg_repack_mlx_affine_switch_gate_up_to_aq_m5": b"qwhip_repack_mlx_affine_switch_gate_up",
    }
    for name, want in table.items():
        assert lib.qwhip_kernel_lookup(name, C.byref(launcher)) == qwhip.OK, name
        assert launcher.value == want
        assert hasattr(lib, want.decode())
    for missing in (b"qwg_gemv_shvq4_g32_v4", b"qwg_gemm_aq7_g32_h16_swiglu", b"qwg_gemv_aq5_g32_v4", b"qwg_head_gemv_shvq4_g32_argmax", b"nope"):
        assert lib.qwhip_kernel_lookup(missing, None) == qwhip.E_KERNEL_MISSING
        assert missing in lib.qwhip_last_error()


def test_status_names_and_null_arguments():
    lib = qwhip.load()
    assert lib.qwhip_status_name(qwhip.OK) == b"ok"
    assert lib.qwhip_status_name(qwhip.E_BAD_WEIGHTS) == b"badWeights"
    assert lib.qwhip_status_name(qwhip.E_KERNEL_MISSING) == b"kernelMissing"
    assert lib.qwhip_device_create(0, None) == qwhip.E_NULL
    assert lib.qwhip_gemv(None, None, None, 0, 1, 0, None, None) == qwhip.E_NULL
    assert lib.qwhip_moe_max_tiles(128, 16384) == min(16384, 128 + 256)
    assert lib.qwhip_moe_max_tiles(128, 8) == 8
    assert lib.qwhip_moe_max_tiles(4, 0) == 0


def test_device_create_fails_loudly_without_a_gpu():
    """No silent CPU fallback: without a gfx950 device the HAL refuses to open."""
    import os
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    lib = qwhip.load()
    h = C.c_void_p()
    assert lib.qwhip_device_create(0, C.byref(h)) == qwhip.E_DEVICE
    assert not h.value
    with pytest.raises(qwhip.QwhipError):
        qwhip.Device(0)


def test_swift_shim_resolves_only_kernel_names_the_library_knows():
    """Every name the Swift shim hands to hal.pipeline() is a key of qwhip_kernel_lookup, so a door of the shim cannot throw
    kernelMissing for a kernel the library serves; the two plan rows whose doors do not exist here (the f16-weight GEMV and the
    MPSGraph prefill door of QWGemm.plan) are the only names without a launcher."""
    import re
    lib = qwhip.load()
    text = (ROOT / "qwegn_amd" / "swift" / "QWHipHAL" / "QWHipHAL.swift").read_text()
    literal = set(re.findall(r'hal\.pipeline\([^"\n]*"([a-z0-9_]+)"', text)) | set(re.findall(r'kernel: "([a-z0-9_]+)"', text))
    literal |= {m for m in re.findall(r'\? "([a-z0-9_]+)" :', text) if m.startswith("qwg_")}
    assert len(literal) >= 20
    missing = {n for n in literal if lib.qwhip_kernel_lookup(n.encode(), None) != qwhip.OK}
    assert missing == {"mpsgraph_bmm_f16", "qwg_gemv_f16_v4"}
    for templ in re.findall(r'"(qwg_[a-z0-9_]*\\\(bank\.bits\)_g\\\(bank\.groupSize\)[a-z0-9_]*)"', text):
        name = templ.replace("\\(bank.bits)", "8").replace("\\(bank.groupSize)", "64")
        assert lib.qwhip_kernel_lookup(name.encode(), None) == qwhip.OK, name
    # the name builders of QWGemmAQ: name("head", bits, group, "tail", isSHVQ) -> head_aq<bits>_g<group>tail
    built = re.findall(r'name\("(qwg_[a-z0-9_]+)", bits, group, "([a-z0-9_]*)", isSHVQ\)', text)
    assert len(built) >= 15
    for head, tail in built:
        name = f"{head}_aq6_g128{tail}"
        assert lib.qwhip_kernel_lookup(name.encode(), None) == qwhip.OK, name
