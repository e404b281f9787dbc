"""CPU-only checks of the C-ABI shared library: it loads, exports every symbol the header declares,
its argument structs have the header's layout, and misuse is rejected with a status code before
anything is launched (no GPU needed)."""

import ctypes
import os
import re
import subprocess

import pytest

from scaling_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355_layer.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return _lib.load()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


def test_exports_match_header(lib):
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS)
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.mi_version() == 100


def test_struct_layout_matches_header(tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include "%s"\n#include <stdio.h>\n#include <stddef.h>\nint main(){printf("%%zu %%zu %%zu %%zu %%zu\\n",'
                   'sizeof(mi_attn_args),sizeof(mi_attn_bwd_args),sizeof(mi_decode_args),'
                   'offsetof(mi_attn_args,stream),offsetof(mi_decode_args,workspace));return 0;}\n' % HEADER)
    exe = tmp_path / "sz"
    subprocess.run(["gcc", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert [int(v) for v in out] == [
        ctypes.sizeof(_lib.MiAttnArgs), ctypes.sizeof(_lib.MiAttnBwdArgs), ctypes.sizeof(_lib.MiDecodeArgs),
        _lib.MiAttnArgs.stream.offset, _lib.MiDecodeArgs.workspace.offset,
    ]


def test_null_and_shape_errors_are_status_codes(lib):
    assert lib.mi_rmsnorm_fwd(None, None, None, None, 4, 64, 1e-5, _lib.MI_BF16, None) == -1
    assert b"null" in lib.mi_last_error()
    assert lib.mi_status_string(-1) == b"MI_E_NULL"
    buf = (ctypes.c_char * 4096)()
    base = ctypes.addressof(buf)
    base += (-base) % 16
    assert lib.mi_rmsnorm_fwd(base, base, base, None, -1, 64, 1e-5, _lib.MI_BF16, None) == -3      # shape
    assert lib.mi_rmsnorm_fwd(base + 2, base, base, None, 4, 64, 1e-5, _lib.MI_BF16, None) == -4   # alignment
    assert lib.mi_swiglu_fwd(None, base, base, 16, _lib.MI_BF16, None) == -1
    assert lib.mi_swiglu_fwd(base, base, base, 0, _lib.MI_BF16, None) == 0                          # empty is fine
    assert lib.mi_rotary(base, base, base, base, None, 4, 2, 8, 3, 16, 8, 16, 8, 4, 4, 0, 0, 0, None) == -3  # odd rot_dim
    assert lib.mi_attn_fwd(None) == -1
    a = _lib.MiAttnArgs()
    assert lib.mi_attn_fwd(ctypes.byref(a)) == 0                                                    # no tokens: nothing to do
    a.total_q = a.total_k = 4
    assert lib.mi_attn_fwd(ctypes.byref(a)) == -1
    a.q = a.k = a.v = a.o = base
    a.cu_seqlens_q = base
    a.dtype = 7
    assert lib.mi_attn_fwd(ctypes.byref(a)) == -2                                                   # unknown dtype code
    a.dtype = _lib.MI_F32                                                                           # float32: its own kernels
    a.head_dim, a.n_q_heads, a.n_kv_heads = 64, 2, 2
    a.rotary_cos = a.rotary_sin = a.position_ids_q = base
    a.total_q = a.total_k = 4
    a.n_docs = 1
    a.q_stride_token = a.k_stride_token = a.v_stride_token = a.o_stride_token = 128
    a.q_stride_head = a.k_stride_head = a.v_stride_head = a.o_stride_head = 64
    a.softmax_scale = 0.125
    a.rotary_table_rows = 4
    assert lib.mi_attn_fwd(ctypes.byref(a)) == -2 and b"rotary" in lib.mi_last_error()              # no fused rotary in fp32
    a.rotary_cos = a.rotary_sin = a.position_ids_q = None
    a.q_stride_head = 62
    assert lib.mi_attn_fwd(ctypes.byref(a)) == -4                                                   # fp32 strides: multiples of 4
    a = _lib.MiAttnArgs()
    a.q = a.k = a.v = a.o = base
    a.cu_seqlens_q = base
    a.total_q = a.total_k = 4
    a.dtype = _lib.MI_BF16
    a.head_dim = 80
    assert lib.mi_attn_fwd(ctypes.byref(a)) == -3
    a.head_dim, a.n_q_heads, a.n_kv_heads = 128, 6, 4
    assert lib.mi_attn_fwd(ctypes.byref(a)) == -3                                                   # heads not divisible
    b = _lib.MiAttnBwdArgs()
    assert lib.mi_attn_bwd(ctypes.byref(b)) == 0                                                    # no tokens
    b.fwd.total_q = b.fwd.total_k = 4
    assert lib.mi_attn_bwd(ctypes.byref(b)) == -1
    d = _lib.MiDecodeArgs()
    assert lib.mi_attn_decode(ctypes.byref(d)) == -1
    assert lib.mi_attn_bwd_workspace_bytes(8192, 32, 128) == 8192 * 32 * 4
    # 8 or more KV heads: nothing to split; one KV head: room for 8 fp32 partial dK and dV next to delta
    assert lib.mi_attn_bwd_workspace_bytes_kv(8192, 8192, 32, 8, 128) == 8192 * 32 * 4
    assert lib.mi_attn_bwd_workspace_bytes_kv(8192, 4096, 32, 1, 128) == 8192 * 32 * 4 + 2 * 8 * 4096 * 128 * 4
    assert lib.mi_attn_decode_static_scratch_bytes() == 8 << 20
    assert lib.mi_attn_decode_static(None) == -1
    assert lib.mi_rmsnorm_bwd_workspace_bytes(8192, 4096) >= 4096 * 4
    assert lib.mi_attn_decode_workspace_bytes(32, 32, 128, 4352) > 0


def test_ops_refuse_to_run_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from scaling_amd import ops
    with pytest.raises(RuntimeError):
        ops.rms_norm(torch.ones(2, 64), torch.ones(64))
