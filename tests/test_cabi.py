"""The C-ABI library loads on a machine without a GPU and exports exactly what the header declares.
No compute entry point is called here."""
import ctypes
import os
import re

from merak_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "merak_tp_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mtp_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared()
    assert len(names) >= 15
    handle = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(handle, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes signatures and header disagree"


def test_loader_and_versions():
    lib = _lib.lib()
    assert lib.mtp_abi_version() == _lib.ABI_VERSION == 12
    hdr = open(os.path.join(ROOT, "include", "merak_tp_gfx950.h")).read()
    assert f"#define MTP_ABI_VERSION {_lib.ABI_VERSION}" in hdr
    for name, val in (("MTP_F32", _lib.MTP_F32), ("MTP_BF16", _lib.MTP_BF16), ("MTP_EPI_NONE", _lib.EPI_NONE),
                      ("MTP_EPI_BIAS", _lib.EPI_BIAS), ("MTP_EPI_BIAS_GELU", _lib.EPI_BIAS_GELU),
                      ("MTP_EPI_SWIGLU", _lib.EPI_SWIGLU), ("MTP_EPI_GELU", _lib.EPI_GELU)):
        assert re.search(rf"#define {name}\s+{val}\b", hdr), name


def test_argument_errors_are_reported_without_a_device():
    lib = _lib.lib()
    # validation happens before any launch: these return error codes on a GPU-less host
    assert lib.mtp_gemv_argmax_workspace_bytes(32, 128256, 4096) == ((128256 + 15) // 16) * 32 * 8
    assert lib.mtp_vocab_ce_fwd(None, None, None, None, None, None, 4, 0, 0, 0, None) == -1
    assert b"vocab" in lib.mtp_last_error()
    assert lib.mtp_linear_fwd(None, None, None, None, None, 4, 4, 4, 7, 0, None) == -1
    assert lib.mtp_gemv(None, None, None, None, 33, 8, 8, 0, 1, None) == -2
    assert b"B=33" in lib.mtp_last_error()
    assert lib.mtp_gemv(None, None, None, None, 4, 8, 8, 0, 0, None) == -2          # fp32 is not a decode dtype
    assert b"dtype 0" in lib.mtp_last_error()
    assert lib.mtp_stream_copy(None, None, 24, None) == -1
    # fused decode GEMV: a norm weight without the sums of squares; K not a multiple of 512; residual with SwiGLU
    assert lib.mtp_gemv_fused(None, None, None, None, 16, None, 1e-5, None, None, None, 0, 1, 64, 512, 0, 1, None) == -1
    assert lib.mtp_gemv_fused(None, None, None, None, 16, 16, 1e-5, None, None, None, 0, 1, 64, 576, 0, 1, None) == -2
    assert b"512" in lib.mtp_last_error()
    assert lib.mtp_gemv_fused(None, None, None, None, None, None, 0.0, 16, None, None, 0, 1, 64, 512, 3, 1, None) == -1


def test_linear_workspace_need_is_zero_for_shapes_that_never_use_scratch():
    lib = _lib.lib()
    full = lib.mtp_linear_workspace_bytes()
    # Llama-3-8B gate/up forward: whole rounds of tiles, no scratch; the Llama-70B shard's o-proj gradients (128
    # tiles, 128 k-tiles each) are what stream-K is for; an fp32 weight gradient with few tiles is cut along k
    assert lib.mtp_linear_workspace_need(0, 4096, 28672, 4096, _lib.MTP_BF16) == 0
    assert lib.mtp_linear_workspace_need(3, 4096, 28672, 4096, _lib.MTP_BF16) == 0
    assert lib.mtp_linear_workspace_need(3, 8192, 8192, 1024, _lib.MTP_BF16) == full
    assert lib.mtp_linear_workspace_need(1, 8192, 8192, 1024, _lib.MTP_F16) == full
    assert lib.mtp_linear_workspace_need(2, 8192, 3072, 768, _lib.MTP_F32) == 8 * (3072 * 768 + 3072) * 4
    assert lib.mtp_linear_workspace_need(0, 8192, 3072, 768, _lib.MTP_F32) == 0
    assert lib.mtp_linear_workspace_need(7, 8, 8, 8, _lib.MTP_BF16) == 0 and lib.mtp_linear_workspace_need(0, 0, 8, 8, 1) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setenv("MERAK_AMD_LIB", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    try:
        _lib.lib()
    except _lib.KernelLibraryMissing as e:
        assert "no CPU/eager fallback" in str(e)
    else:
        raise AssertionError("a missing kernel library must raise")
