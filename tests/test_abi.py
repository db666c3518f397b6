"""CPU-side checks of the C ABI: the library loads and exports every symbol
include/moa_hip.h declares; host-only entry points behave; the package refuses
to run without its library or on CPU tensors.  No kernel is launched."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from moa_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build()
    return _lib.load()


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "moa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moa_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_exported(lib):
    from moa_amd import _lib
    names = _declared_symbols()
    assert len(names) >= 8
    assert sorted(_lib.SIGNATURES) == names, "python binding and header disagree"
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n


def test_host_only_entry_points(lib):
    assert lib.moa_abi_version() == 1
    # decode workspace: (ceil(sumC/256) + Hkv) * (Hq/Hkv) partial slots per batch row, D+2 floats each,
    # rounded up to 256 bytes
    def expect(B, Hq, Hkv, D, sumC):
        raw = B * (-(-sumC // 256) + Hkv) * (Hq // Hkv) * (D + 2) * 4
        return -(-raw // 256) * 256
    assert lib.moa_decode_workspace_bytes(2, 4, 4, 128, 1024) == expect(2, 4, 4, 128, 1024)
    assert lib.moa_decode_workspace_bytes(3, 16, 2, 64, 5000) == expect(3, 16, 2, 64, 5000)
    assert lib.moa_decode_workspace_bytes(0, 4, 4, 128, 1024) == 0
    assert lib.moa_cache_prefill_workspace_bytes(3, 100) >= 3 * 201 * 4


def test_argument_errors_without_gpu(lib):
    from moa_amd import _lib
    # null pointers are rejected before anything is launched
    rc = lib.moa_decode_fwd(None, None, None, None, None, 0, None, None, 1, 1, 1, 128, 64, 1.0, 0, None)
    assert rc == _lib.MOA_ERR_ARG and "null" in _lib.last_error()
    rc = lib.moa_cache_append(None, None, None, None, None, None, None, None, None, None, None, None, None,
                              0, 1, 1, 128, 64, 0, None)
    assert rc == _lib.MOA_ERR_ARG
    with pytest.raises(AssertionError):
        _lib.check(_lib.MOA_ERR_ARG)
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.MOA_ERR_UNSUPPORTED)


def test_prefill_size_limits_without_gpu(lib):
    """Sizes beyond what the prefill work queue's ticket arithmetic covers are refused before anything is
    launched or looked up on a device (include/moa_hip.h): more than 2^22 (batch, head) pairs, more than
    2^25 work items, a prompt longer than 2^28."""
    from moa_amd import _lib
    I4 = ctypes.c_int64 * 4
    p = ctypes.c_void_p(0x10000)   # never dereferenced: the call fails on the sizes
    for B, Hq, N in (((1 << 20), 8, 64), (1 << 16, 8, 1 << 15), (8, 8, 1 << 29)):
        D = 64
        st = I4(Hq * N * D, N * D, D, 1)
        rc = lib.moa_prefill_fwd(p, p, p, p, st, st, st, st, B, Hq, Hq, N, D, p, p, 0.1, _lib.MOA_DTYPE_F16, None)
        assert rc == _lib.MOA_ERR_UNSUPPORTED and "too many work items" in _lib.last_error(), (B, Hq, N)


def test_no_cpu_path():
    from moa_amd import StaticCircularCache, _lib, mixture_of_sparse_attention
    q = torch.zeros(1, 2, 1, 128, dtype=torch.float16)
    k = torch.zeros(1, 256, 128, dtype=torch.float16)
    hs = torch.tensor([[0, 128]])
    hv = torch.tensor([[128, 128]])
    with pytest.raises(_lib.MoaKernelError):
        mixture_of_sparse_attention(q, k, k, 1.0, head_start_index=hs, head_valid_length=hv)
    qp = torch.zeros(1, 2, 128, 64, dtype=torch.float16)
    with pytest.raises(_lib.MoaKernelError):
        mixture_of_sparse_attention(qp, qp, qp, 1.0, sink_size=torch.tensor([64, 64]), local_size=torch.tensor([64, 64]))
    c = StaticCircularCache([[128, 128]], static_size=[[64, 64]], batch_size=1, head_dim=64)
    with pytest.raises(_lib.MoaKernelError):
        c.update(qp, qp, 0)


def test_invalid_input_raises_assertion():
    """The reference's test_invalid_input (tests/attention_kernel_test.py:140-149)."""
    from moa_amd import mixture_of_sparse_attention
    q = torch.rand(2, 4, 10, 64, dtype=torch.float16)
    k = torch.rand(2, 4, 10, 65, dtype=torch.float16)
    v = torch.rand(2, 4, 10, 64, dtype=torch.float16)
    with pytest.raises(AssertionError):
        mixture_of_sparse_attention(q, k, v, 0.1)


def test_missing_library_is_loud(monkeypatch, tmp_path):
    from moa_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmoa_hip.so"))
    with pytest.raises(_lib.MoaKernelError):
        _lib.load()


def test_python_constants_match_the_header():
    """The size limit of the entry point that allocates nothing is written down twice (header and
    _lib.py): the two must agree."""
    import re
    from moa_amd import _lib
    text = open(os.path.join(ROOT, "include", "moa_hip.h")).read()
    m = re.search(r"#define\s+MOA_DECODE_NOALLOC_MAX_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", text)
    assert m, "MOA_DECODE_NOALLOC_MAX_BYTES not found in the header"
    assert int(m.group(1)) << int(m.group(2)) == _lib.MOA_DECODE_NOALLOC_MAX_BYTES
    for name in ("MOA_OK", "MOA_ERR_ARG", "MOA_ERR_UNSUPPORTED", "MOA_ERR_LAUNCH", "MOA_ERR_WORKSPACE",
                 "MOA_DTYPE_F16", "MOA_DTYPE_BF16", "MOA_DTYPE_F32"):
        m = re.search(r"#define\s+%s\s+\(?(-?\d+)\)?" % name, text) or re.search(r"%s\s*=\s*(-?\d+)" % name, text)
        assert m, name
        assert int(m.group(1)) == getattr(_lib, name), name
