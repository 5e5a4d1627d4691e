"""Drop-in surface: names, signatures, defaults and routing of the reference package
(adasplash/__init__.py:1-85, tests/test_public_api.py:7-50), host-side argument checks, and the C ABI."""

import ctypes
import inspect
import re
from pathlib import Path

import pytest
import torch

import adasplash_amd
from adasplash_amd import _lib

ROOT = Path(__file__).resolve().parents[1]


def test_exports_are_lazy_and_versioned():
    assert adasplash_amd.__version__ == "0.2.0"
    for name in ["adasplash", "adasplash_v1", "adasplash_v2", "adasplash_no_block_mask", "triton_entmax",
                 "triton_entmax_v1", "triton_entmax_v2", "triton_sparsemax", "triton_entmax15", "adasplash2"]:
        assert name in adasplash_amd.__all__
        assert callable(getattr(adasplash_amd, name))
    assert not hasattr(adasplash_amd, "entmax_attention")


def test_signatures_and_defaults():
    sig = inspect.signature
    assert str(sig(adasplash_amd.adasplash)) == "(q, k, v, alpha=1.5, is_causal=True, varlen=None, niter=None)"
    assert str(sig(adasplash_amd.adasplash_v1)) == "(q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10)"
    assert str(sig(adasplash_amd.adasplash_v2)) == "(q, k, v, niter=1, varlen=None)"
    assert str(sig(adasplash_amd.triton_entmax)) == "(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False)"
    assert str(sig(adasplash_amd.triton_entmax_v2)) == "(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False)"
    assert str(sig(adasplash_amd.triton_entmax_v1)) == "(x, alpha=1.5, n_iter=10, fast_math=True)"


def test_dispatcher_is_not_shadowed_by_submodules():
    import adasplash_amd.adasplash_v2  # noqa: F401
    import adasplash_amd.triton_entmax_v2  # noqa: F401

    assert callable(adasplash_amd.adasplash_v2) and callable(adasplash_amd.triton_entmax_v2)
    assert list(inspect.signature(adasplash_amd.adasplash_v2).parameters) == ["q", "k", "v", "niter", "varlen"]


def test_dispatcher_routing(monkeypatch):
    calls = []
    import adasplash_amd.adasplash_block_mask as v1mod
    import adasplash_amd.adasplash_v2 as v2mod

    monkeypatch.setattr(v1mod, "sparse_attn", lambda q, k, v, **kw: calls.append(("v1", kw)))
    monkeypatch.setattr(v2mod, "sparse_attn", lambda q, k, v, **kw: calls.append(("v2", kw)))
    adasplash_amd.adasplash(1, 2, 3)
    adasplash_amd.adasplash(1, 2, 3, alpha=1.333)
    adasplash_amd.adasplash(1, 2, 3, is_causal=False)
    adasplash_amd.adasplash(1, 2, 3, niter=4)
    adasplash_amd.adasplash(1, 2, 3, alpha=2.0, niter=3)
    assert calls[0] == ("v2", {"niter": 1, "varlen": None})
    assert calls[1] == ("v1", {"alpha": 1.333, "is_causal": True, "varlen": None, "niter": 10})
    assert calls[2] == ("v1", {"alpha": 1.5, "is_causal": False, "varlen": None, "niter": 10})
    assert calls[3] == ("v2", {"niter": 4, "varlen": None})
    assert calls[4][0] == "v1" and calls[4][1]["niter"] == 3


def test_entmax_argument_fixups(monkeypatch):
    import adasplash_amd.triton_entmax_v2 as mod

    seen = []
    monkeypatch.setattr(mod._EntmaxRows, "apply", staticmethod(lambda *a: seen.append(a)))
    mod.triton_entmax("x", alpha=1.333, n_iter=2)
    mod.triton_entmax("x", alpha=1.5)
    mod.triton_sparsemax("x", n_iter=5)
    mod.triton_entmax15("x")
    assert seen[0] == ("x", 1.333, 10, False, False)  # no histogram, at least 10 steps
    assert seen[1] == ("x", 1.5, 2, True, False)
    assert seen[2] == ("x", 2.0, 5, True, False)
    assert seen[3] == ("x", 1.5, 2, True, False)


# ---- host-side checks fire before anything touches a device (adasplash_v2.py:1248-1276) ---------------
def _qkv(B=1, H=2, N=128, D=32, Hkv=None):
    Hkv = H if Hkv is None else Hkv
    return torch.zeros(B, H, N, D), torch.zeros(B, Hkv, N, D), torch.zeros(B, Hkv, N, D)


def test_v2_rejects_bad_arguments():
    q, k, v = _qkv(D=24)
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q, k, v)
    q, k, v = _qkv(N=32)
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q, k, v)
    q, k, v = _qkv(N=96)
    with pytest.raises(AssertionError):  # not a power of two without varlen
        adasplash_amd.adasplash_v2(q, k, v)
    q, k, v = _qkv(H=3, Hkv=2)
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q, k, v)
    q, k, v = _qkv()
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q.transpose(1, 2).contiguous().transpose(1, 2), k, v)
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q, k, v, varlen=torch.tensor([[128]]))
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q, k, v, varlen=torch.tensor([128.0]))
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v2(q, k, v[:, :, :64])


def test_v1_and_entmax_reject_bad_arguments():
    q, k, v = _qkv(N=96)
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v1(q, k, v)
    q, k, v = _qkv(D=48)
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v1(q, k, v)
    q, k, v = _qkv()
    with pytest.raises(AssertionError):
        adasplash_amd.adasplash_v1(q, k, v, varlen=torch.tensor([[1]]))
    with pytest.raises(AssertionError):
        adasplash_amd.triton_entmax(torch.zeros(4, 8).t())


def test_there_is_no_cpu_fallback():
    q, k, v = _qkv()
    with pytest.raises(RuntimeError, match="ROCm device"):
        adasplash_amd.adasplash_v2(q, k, v)
    with pytest.raises(RuntimeError, match="ROCm device"):
        adasplash_amd.adasplash_v1(q, k, v)
    with pytest.raises(RuntimeError, match="ROCm device"):
        adasplash_amd.triton_entmax(torch.zeros(2, 8))


def test_package_never_imports_the_oracle():
    for path in (ROOT / "adasplash_amd").rglob("*.py"):
        assert not re.search(r"^\s*(from|import)\s+oracle", path.read_text(), re.M), path


# ---- C ABI -----------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "adasplash_hip.h").read_text()
    declared = set(re.findall(r"\b(adsp_[a-z0-9_]+)\s*\(", header))
    assert {"adsp_entmax_rows_fwd", "adsp_attn_v2_fwd", "adsp_attn_v1_fwd", "adsp_attn_workspace_bytes"} <= declared
    lib = ctypes.CDLL(str(_lib.lib_path()))
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/adasplash_hip.h but not exported"


def test_library_is_built_from_the_sources_in_the_tree():
    """The library carries a hash of the kernel sources, headers and flags it was built from; a library older than
    the sources beside it must not pass for them."""
    from adasplash_amd import build

    lib = ctypes.CDLL(str(_lib.lib_path()))
    lib.adsp_build_id.restype = ctypes.c_char_p
    have = lib.adsp_build_id().decode()
    assert re.fullmatch(r"[0-9a-f]{16}", have), have
    lib.adsp_build_flags.restype = ctypes.c_char_p
    flags = lib.adsp_build_flags().decode()  # the extra flags of a profiling build (empty otherwise) enter the id
    assert have == build.source_id(flags), "libadasplash_hip.so is stale: run `python -m adasplash_amd.build`"
    assert build.source_id("-DADSP_SPARSE_STOP=1") != build.source_id("")
    assert _lib.build_id() == have  # and the loader, which makes the same comparison, accepts it


def test_sizing_helpers_and_status_strings():
    lib = _lib.load()
    assert lib.adsp_version() >= 1
    # head dims the sparse-support kernel does not serve need no workspace ...
    assert lib.adsp_attn_workspace_bytes(2, 2, 2, 100, 32, _lib.ADSP_F16) == 0
    # ... and at head dims 64 / 128 it holds that kernel's counters, flags, candidate slots (at most 1024) and copy of K
    slot = 4 * 1616 * 8
    k8 = 8 * 8 * 8192 * 128  # the one-byte copy of K
    assert lib.adsp_attn_workspace_bytes(8, 32, 8, 8192, 128, _lib.ADSP_BF16) == 256 + 1792 + 8 * 32 * 64 * 4 + 1024 * slot + k8  # (8 * 8 + 1) word pairs and four floats per K/V head, padded to 256
    small = lib.adsp_attn_workspace_bytes(1, 2, 2, 128, 64, _lib.ADSP_F16)
    assert 8 * slot < small < 8 * slot + 2 * 64 * 128 * 3 + 1024
    assert lib.adsp_attn_workspace_bytes(8, 32, 8, 8192, 128, _lib.ADSP_F32) == 0
    assert lib.adsp_attn_bmask_words(8192) == 64 * 4 and lib.adsp_attn_bmask_words(64) == 1
    # supports kept for the backward: per 128-row block of a query head a flag, four stream lengths and the four
    # streams, plus a word per row; nothing where the sparse-support kernel does not run
    items = 8 * 32 * 64
    assert lib.adsp_attn_supports_bytes(8, 32, 8, 8192, 128, _lib.ADSP_BF16) == items * 4 + items * 8 + 8 * 32 * 8192 * 4 + items * slot
    assert lib.adsp_attn_supports_bytes(8, 32, 8, 8192, 128, _lib.ADSP_F32) == 0
    assert lib.adsp_attn_supports_bytes(2, 2, 2, 100, 32, _lib.ADSP_F16) == 0
    assert lib.adsp_attn_bwd_workspace_bytes(8, 32, 8, 8192, 128, _lib.ADSP_BF16) > 2 * 8 * 32 * 8192 * 128 * 4 + items * slot
    # with a causal mask the later key blocks need no partial rows: 5/16 of them are left
    any_mask = lib.adsp_attn_bwd_workspace_bytes(8, 32, 8, 8192, 128, _lib.ADSP_BF16)
    assert lib.adsp_attn_bwd_workspace_bytes_causal(8, 32, 8, 8192, 128, _lib.ADSP_BF16, 0) == any_mask
    assert lib.adsp_attn_bwd_workspace_bytes_causal(8, 32, 8, 8192, 128, _lib.ADSP_BF16, 1) == any_mask - 2 * 8 * 32 * (8192 - 2560) * 128 * 4
    assert lib.adsp_attn_bwd_workspace_bytes_causal(8, 8, 8, 8192, 128, _lib.ADSP_BF16, 1) == lib.adsp_attn_bwd_workspace_bytes(8, 8, 8, 8192, 128, _lib.ADSP_BF16)
    assert lib.adsp_status_string(0) == b"ok"
    assert all(len(lib.adsp_status_string(s)) > 0 for s in range(0, 9))


def test_backward_workspace_for_a_causal_call_follows_the_merge_border(monkeypatch):
    """With a causal mask and several query heads per K/V head the partial rows cover the key blocks in front of
    N * ADSP_DKDV_MERGE256 / 256 only (rounded up to whole 128-key blocks); the rest of the workspace is the same."""
    lib = _lib.load()
    B, Hq, Hkv, D = 2, 8, 2, 64
    for N in (128, 1000, 4096, 8192, 65536):
        for m256 in (0, 1, 64, 80, 200, 256):
            monkeypatch.setenv("ADSP_DKDV_MERGE256", str(m256))
            full = lib.adsp_attn_bwd_workspace_bytes(B, Hq, Hkv, N, D, _lib.ADSP_BF16)
            causal = lib.adsp_attn_bwd_workspace_bytes_causal(B, Hq, Hkv, N, D, _lib.ADSP_BF16, 1)
            rows = N
            if m256 > 0:
                bound = (N * m256 + 255) // 256
                rows = min(N, (bound + 127) // 128 * 128)
            assert full - causal == 2 * B * Hq * (N - rows) * D * 4, (N, m256)
            assert lib.adsp_attn_bwd_workspace_bytes_causal(B, Hq, Hkv, N, D, _lib.ADSP_BF16, 0) == full
            assert lib.adsp_attn_bwd_workspace_bytes_causal(B, Hq, Hq, N, D, _lib.ADSP_BF16, 1) == lib.adsp_attn_bwd_workspace_bytes(B, Hq, Hq, N, D, _lib.ADSP_BF16)


def test_argument_errors_come_back_as_status_codes():
    lib = _lib.load()
    # no pointer is dereferenced and nothing is launched for these
    assert lib.adsp_entmax_rows_fwd(None, None, 4, 8, 0, 1.5, 2, 1, 0, None) == 1
    assert lib.adsp_entmax_rows_fwd(None, None, 0, 8, 0, 1.5, 2, 1, 0, None) == 0
    assert lib.adsp_entmax_rows_fwd(16, 16, 4, 8, 9, 1.5, 2, 1, 0, None) == 3
    assert lib.adsp_entmax_rows_fwd(16, 16, 4, 8, 0, 1.0, 2, 1, 0, None) == 5
    assert lib.adsp_attn_v2_fwd(None, None, None, None, None, None, None, 0, 1, 1, 1, 64, 64, 1, 1, None, 0, None) == 1
    assert lib.adsp_attn_v2_fwd(16, 16, 16, 16, None, None, None, 0, 1, 3, 2, 64, 64, 1, 1, None, 0, None) == 2
    assert lib.adsp_attn_v2_fwd(16, 16, 16, 16, None, None, None, 0, 1, 1, 1, 64, 48, 1, 1, None, 0, None) == 2
    assert lib.adsp_attn_v2_fwd(16, 16, 16, 8, None, None, None, 0, 1, 1, 1, 64, 64, 1, 1, None, 0, None) == 4
    assert lib.adsp_attn_v2_fwd(16, 16, 16, 16, None, None, None, 0, 1, 1, 1, 64, 64, 1, 1, None, 0, None) == 6
    assert lib.adsp_attn_v1_fwd(16, 16, 16, 16, None, None, None, 0, 1, 1, 64, 64, 0, 2.5, 0, 1, None, 0, None,
                                None) == 5


def test_dense_example_names_and_signatures():
    """``examples/attention.py:34-44,94``: the dense path and the dispatcher alias keep their argument lists."""
    import inspect

    from adasplash_amd import dense

    sig = inspect.signature(dense.slow_entmax_attention)
    assert list(sig.parameters) == ["q", "k", "v", "alpha", "varlen", "is_causal", "padding", "niter", "alibi_slopes"]
    assert [sig.parameters[n].default for n in ("alpha", "varlen", "is_causal", "padding", "niter", "alibi_slopes")] == \
        [1.5, None, False, "right", 2, None]
    sig = inspect.signature(dense.flash_entmax_attention)
    assert list(sig.parameters) == ["q", "k", "v", "alpha", "varlen", "is_causal", "niter"]
    assert sig.parameters["is_causal"].default is True


def test_keep_supports_modes():
    """What the forward keeps for the backward is a mode of the package, not an environment variable only."""
    import torch

    import adasplash_amd
    from adasplash_amd import _attention

    old = adasplash_amd.set_keep_supports("never")
    try:
        assert old in ("auto", "always", "never")
        q = torch.zeros(1, 2, 1024, 64, dtype=torch.bfloat16)  # 256 KB
        assert not _attention._keeps(1 << 20, q)
        adasplash_amd.set_keep_supports("always")
        assert _attention._keeps(1 << 40, q) and not _attention._keeps(0, q)
        adasplash_amd.set_keep_supports("auto")
        assert _attention._keeps(256 << 20, q) and not _attention._keeps((256 << 20) + 1, q)
        big = torch.zeros(1, 1, 1, 1, dtype=torch.bfloat16).expand(8, 32, 8192, 128)  # the headline q: 512 MiB
        assert _attention._keeps(860 << 20, big) and not _attention._keeps(1100 << 20, big)
        with pytest.raises(ValueError):
            adasplash_amd.set_keep_supports("sometimes")
    finally:
        adasplash_amd.set_keep_supports(old)
