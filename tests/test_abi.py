"""The C-ABI library on a machine without a GPU: it loads, exports every declared symbol, and
its host-side argument checks report errors the way the header promises."""
import ctypes as C
import os
import re

import pytest

from tests.conftest import ROOT


@pytest.fixture(scope="module")
def lib():
    from vui_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libvui_amd.so not built (python -m vui_amd.build)")
    return _lib.load()


def declared_functions():
    inc = os.path.join(ROOT, "include")
    src = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(vui_[a-z0-9_]+)\s*\(", src)))


def test_header_and_binding_agree(lib):
    from vui_amd import _lib

    names = declared_functions()
    assert names, "no declarations found"
    assert sorted(_lib.SIGNATURES) == names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared but not exported"


def nano_cfg():
    from vui_amd import _lib

    c = _lib.VuiConfigC()
    c.dtype, c.d_model, c.n_layers, c.n_heads, c.n_kv_heads, c.head_dim, c.ffn = 0, 768, 22, 8, 8, 96, 2048
    c.n_quantizers, c.codebook_size, c.rq_dim, c.rq_layers, c.rq_heads, c.rq_ffn = 16, 2048, 512, 4, 8, 1408
    c.rope_dim, c.max_seqlen, c.n_slots, c.window, c.norm_eps, c.rq_norm_eps = 96, 4608, 2, 0, 1e-5, 1e-6
    return c


def test_sizes(lib):
    c = nano_cfg()
    assert lib.vui_kv_bytes(C.byref(c)) == 22 * 2 * 4608 * 8 * 96 * 2
    n1, n16 = lib.vui_workspace_bytes(C.byref(c), 1), lib.vui_workspace_bytes(C.byref(c), 16)
    # the workspace of a bf16 context also holds the layers' projection weights in the prefill pass's operand layout
    tiled = 22 * (2304 * 768 + 768 * 768 + 2 * 2048 * 768 + 768 * 2048) * 2
    # ... and the depth head's matrices in the batched kernel's layout (4 layers, 15 codebook heads, the projection)
    tiled += (4 * (4 * 512 * 512 + 3 * 1408 * 512) + 15 * 2048 * 512 + 512 * 768) * 2
    assert 0 < n1 < n16 and tiled < n1 and n16 - tiled < 64 << 20
    assert lib.vui_attn_scratch_bytes(1, 8, 96, 32) >= 8 * 32 * 98 * 4
    assert lib.vui_version() >= 1


def test_argument_errors(lib):
    from vui_amd import _lib

    c = nano_cfg()
    assert lib.vui_workspace_bytes(C.byref(c), 17) < 0
    assert "max_batch" in _lib.last_error()
    c.head_dim = 100  # H * hd != d
    assert lib.vui_workspace_bytes(C.byref(c), 1) < 0
    assert "head layout" in _lib.last_error()
    c = nano_cfg()
    w = _lib.WeightsC()
    h = C.c_void_p()
    buf = (C.c_char * 4096)()
    rc = lib.vui_ctx_create(C.byref(c), C.byref(w), C.addressof(buf), 4096, 1, C.byref(h))
    assert rc == -12 and "workspace too small" in _lib.last_error()
    rc = lib.vui_backbone_step(None, None, None, None, None, None, 1, None, None, None, None, None, 1, None)
    assert rc == -22 and "NULL context" in _lib.last_error()
    with pytest.raises(RuntimeError, match="NULL graph"):
        _lib.check(lib.vui_graph_launch(None, None), "vui_graph_launch")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from vui_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()
