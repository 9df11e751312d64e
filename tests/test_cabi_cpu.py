"""Host-side checks that need no GPU: the shared library loads, exports every symbol the header
declares, agrees with the Python binding on the struct layout, and fa_validate returns the
documented code for each malformed argument.  The operator's Python layer raises the same
AssertionErrors as the reference (flash_triton.py:510-530) before touching the GPU."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

from flash_mi355 import _cabi, attention, SCORE_FUNC_MODE1_DOC

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "flash_mi355.h").read_text()


def _declared_functions():
    body = HEADER.split('extern "C" {')[1]
    return sorted(set(re.findall(r"^\s*(?:const\s+)?[a-z_0-9]+\*?\s+(fa_[a-z_0-9]+)\s*\(", body, re.M)))


def test_library_exports_every_declared_symbol():
    L = _cabi.lib()
    names = _declared_functions()
    assert set(names) == set(_cabi.EXPORTS), (names, _cabi.EXPORTS)
    for n in names:
        assert getattr(L, n) is not None


def test_clock_stamp_build_is_a_library_of_its_own():
    """bench.py --wg-trace loads libflash_mi355_trace.so: every entry point of the header plus
    fa_trace_read.  The product library carries no trace export."""
    from flash_mi355.build import TRACE_LIB_PATH
    assert TRACE_LIB_PATH.exists(), "python -m flash_mi355.build builds it next to the product library"
    T = ctypes.CDLL(str(TRACE_LIB_PATH))
    for n in _declared_functions() + ["fa_trace_read"]:
        assert getattr(T, n) is not None
    T.fa_version.restype = ctypes.c_int
    assert T.fa_version() == _cabi.FA_ABI_VERSION
    with pytest.raises(AttributeError):
        _cabi.lib().fa_trace_read


def test_struct_layout_and_version():
    L = _cabi.lib()
    assert L.fa_version() == _cabi.FA_ABI_VERSION == int(re.search(r"#define FA_ABI_VERSION (\d+)", HEADER).group(1))
    assert L.fa_params_size() == ctypes.sizeof(_cabi.FaParams)
    for code in range(0, -11, -1):
        assert L.fa_error_string(code)


def _good_params(buf):
    p = _cabi.FaParams()
    base = (ctypes.addressof(buf) + 255) & ~255
    for f in ("q", "k", "v", "o", "lse", "dout", "dq", "dk", "dv", "delta"):
        setattr(p, f, base)
    p.B, p.H, p.Hk, p.M, p.N, p.D = 1, 4, 2, 128, 256, 64
    for f in ("q_stride", "o_stride", "do_stride", "dq_stride"):
        arr = getattr(p, f); arr[0], arr[1], arr[2], arr[3] = 4 * 128 * 64, 128 * 64, 64, 1
    for f in ("k_stride", "v_stride", "dk_stride", "dv_stride"):
        arr = getattr(p, f); arr[0], arr[1], arr[2], arr[3] = 4 * 256 * 64, 256 * 64, 64, 1
    p.causal, p.score_mode, p.dtype, p.sm_scale = 1, 0, _cabi.FA_DTYPE_BF16, 0.125
    return p


def test_validate_codes():
    L = _cabi.lib()
    buf = ctypes.create_string_buffer(4096)
    v = lambda p, stage=1: L.fa_validate(ctypes.byref(p), stage)
    assert v(_good_params(buf)) == 0
    assert L.fa_validate(None, 0) == -1
    p = _good_params(buf); p.D = 48; assert v(p) == -2           # flash_triton.py:512
    p = _good_params(buf); p.D = 256; assert v(p) == -2
    p = _good_params(buf); p.dtype = 5; assert v(p) == -3
    p = _good_params(buf); p.H = 3; assert v(p) == -4             # H % Hk, flash_triton.py:518
    p = _good_params(buf); p.M, p.N = 256, 128; assert v(p) == -4  # causal needs N >= M, flash_triton.py:520
    p = _good_params(buf); p.M, p.N, p.causal = 256, 128, 0; assert v(p) == 0
    p = _good_params(buf); p.B = 0; assert v(p) == -4
    p = _good_params(buf); p.q += 8; assert v(p) == -5
    p = _good_params(buf); p.q_stride[2] = 68; assert v(p) == -5
    p = _good_params(buf); p.k_stride[3] = 2; assert v(p) == -6
    p = _good_params(buf); p.score_mode = 3; assert v(p) == -7
    p = _good_params(buf); p.score_mode = 1; assert v(p) == -7     # doc mode without ids
    p = _good_params(buf); p.score_mode = 1; p.eq = p.ek = p.q; assert v(p) == -8   # no workspace
    p = _good_params(buf); p.dout = None; assert v(p, 1) == -1 and v(p, 0) == 0
    p = _good_params(buf); p.flags = 2; assert v(p) == -7
    # the diagnostic flag of the dk/dv pair wait is honoured by fa_bwd_dkdv's stage alone
    p = _good_params(buf); p.flags = _cabi.FA_FLAG_DEBUG_NO_PAIR_WAIT
    assert v(p, 3) == 0 and v(p, 0) == -7 and v(p, 1) == -7 and v(p, 2) == -7
    p = _good_params(buf); p.dout = None; assert v(p, 3) == -1
    # per-row causal positions: only with causal + ids, not with a prefix; they lift the N >= M rule
    p = _good_params(buf); p.qpos = p.q; assert v(p) == -7           # no ids
    p = _good_params(buf); p.qpos = p.q; p.score_mode = 1; p.eq = p.ek = p.q; p.causal = 0; assert v(p, 2) == -7
    p = _good_params(buf); p.qpos = p.q; p.score_mode = 1; p.eq = p.ek = p.q; p.prefix = 4; assert v(p, 2) == -7
    p = _good_params(buf); p.qpos = p.q; p.score_mode = 1; p.eq = p.ek = p.q; p.M, p.N = 256, 128; assert v(p, 2) == -8   # past the shape check: no workspace
    p = _good_params(buf); p.flags = _cabi.FA_FLAG_DQ_DELTA; assert v(p) == 0 and v(p, 1) == 0
    p = _good_params(buf); p.flags = _cabi.FA_FLAG_DQ_DELTA; p.dtype = _cabi.FA_DTYPE_FP32; assert v(p, 1) == 0
    # block mask: eq carries the byte map, no workspace, no ek; rows of the map at least ceil(N/64) apart
    p = _good_params(buf); p.score_mode = _cabi.FA_SCORE_MODE2_BLOCK; assert v(p) == -7
    p = _good_params(buf); p.score_mode = _cabi.FA_SCORE_MODE2_BLOCK; p.eq = p.q; p.eq_stride[2] = (p.N + 63) // 64
    assert v(p) == 0 and L.fa_workspace_bytes(ctypes.byref(p)) == 0
    p.eq_stride[2] -= 1; assert v(p) == -6
    p.eq_stride[2] += 1; p.dtype = _cabi.FA_DTYPE_FP32; assert v(p) == 0
    # sliding window / prefix: causal only, not both, not negative
    p = _good_params(buf); p.window = 64; assert v(p) == 0
    p = _good_params(buf); p.prefix = 64; assert v(p) == 0
    p = _good_params(buf); p.window = 64; p.prefix = 8; assert v(p) == -7
    p = _good_params(buf); p.window = -1; assert v(p) == -7
    p = _good_params(buf); p.M, p.N, p.causal, p.window = 256, 128, 0, 16; assert v(p) == -7
    # fp32 tensors are accepted; their strides must be multiples of 16 bytes = 4 elements
    p = _good_params(buf); p.dtype = _cabi.FA_DTYPE_FP32; assert v(p) == 0
    p = _good_params(buf); p.dtype = _cabi.FA_DTYPE_FP32; p.q_stride[2] = 68; assert v(p) == 0
    p = _good_params(buf); p.dtype = _cabi.FA_DTYPE_FP32; p.q_stride[2] = 66; assert v(p) == -5


def test_workspace_size():
    L = _cabi.lib()
    buf = ctypes.create_string_buffer(4096)
    p = _good_params(buf)
    assert L.fa_workspace_bytes(ctypes.byref(p)) == 0
    p.score_mode = 1
    p.eq_stride[0], p.eq_stride[1], p.eq_stride[2] = 128, 0, 1       # ids shared by the heads
    p.ek_stride[0], p.ek_stride[1], p.ek_stride[2] = 4 * 256, 256, 1   # per head
    r256 = lambda x: (x + 255) // 256 * 256
    Pp = 256 + 256
    want = (r256(128 * 4) + r256(4 * 256 * 4) + 3 * r256(Pp * 4) + r256(4) + r256(32) + r256(Pp // 64 * 32)
            + r256(4 * 4 * 32))
    assert L.fa_workspace_bytes(ctypes.byref(p)) == want   # 4 key tiles of 64: no key range is ever split
    assert L.fa_workspace_plan_bytes(ctypes.byref(p)) == want   # ... so all of it is plan
    # from 32 key tiles on, scratch for split global-row tiles: arrival counters, (max, sum) pairs, fp32
    # partial tiles; chunks = clamp(key tiles / 32, 2, 4) (finer when the launch is short of workgroups),
    # splittable tiles = min(128 MiB / footprint, 64), at most ceil(M / 128) + 1
    p.N = 2048
    p.ek_stride[0], p.ek_stride[1] = 4 * 2048, 2048
    chunks, tiles = 2, 2   # 32 key tiles -> 2 chunks of 16; M = 128 rows -> 2 tiles
    assert p.M == 128 and (128 << 20) // (1 * 4 * chunks * 128 * (p.D + 2) * 4) >= 64
    want = (r256(128 * 4) + r256(4 * 2048 * 4) + 3 * r256(Pp * 4) + r256(4) + r256(32) + r256(Pp // 64 * 32)
            + r256(4 * 32 * 32)
            + r256(4 * tiles * 4) + r256(4 * tiles * chunks * 128 * 2 * 4) + r256(4 * tiles * chunks * 128 * p.D * 4))
    assert L.fa_workspace_bytes(ctypes.byref(p)) == want
    # the plan proper (what has to survive from forward to backward) ends after the counters
    scratch = r256(4 * tiles * chunks * 128 * 2 * 4) + r256(4 * tiles * chunks * 128 * p.D * 4)
    assert L.fa_workspace_plan_bytes(ctypes.byref(p)) == want - scratch


def test_python_layer_asserts_like_the_reference():
    q = torch.zeros(1, 4, 8, 64, dtype=torch.bfloat16)
    k = torch.zeros(1, 2, 16, 64, dtype=torch.bfloat16)
    e_q = torch.zeros(1, 4, 8, dtype=torch.int32)
    with pytest.raises(AssertionError):
        attention(q, k, torch.zeros(1, 2, 16, 32, dtype=torch.bfloat16))          # feature sizes differ
    with pytest.raises(AssertionError):
        attention(torch.zeros(1, 4, 8, 48), torch.zeros(1, 2, 16, 48), torch.zeros(1, 2, 16, 48))   # D not in {16,32,64,128}
    with pytest.raises(AssertionError):
        attention(q, k, torch.zeros(1, 1, 16, 64, dtype=torch.bfloat16))          # kv head counts differ
    with pytest.raises(AssertionError):
        attention(torch.zeros(1, 3, 8, 64), k, k)                                   # H % Hk
    with pytest.raises(AssertionError):
        attention(torch.zeros(1, 4, 32, 64, dtype=torch.bfloat16), k, k, causal=True)   # causal with N < M
    with pytest.raises(AssertionError):
        attention(q, k, k, eq=e_q)                                                  # eq without ek
    with pytest.raises(AssertionError):
        attention(q, k, k, score_func_mode=SCORE_FUNC_MODE1_DOC)                    # doc mode without ids
    with pytest.raises(AssertionError):
        attention(q, k, k)                                                          # CPU tensors: no CPU fallback


def test_operands_on_another_device_are_refused():
    """Ids, k, v or dO that do not live on q's device are refused with an AssertionError before any
    pointer reaches a kernel (checked on the helper itself: no GPU is needed to compare devices)."""
    from flash_mi355 import api
    q = torch.zeros(1, 1, 8, 16, device="meta")
    api._check_same_device(q, k=torch.zeros(2, device="meta"), eq=None)
    with pytest.raises(AssertionError, match="eq is on cpu"):
        api._check_same_device(q, eq=torch.zeros(1, 1, 8, dtype=torch.int32))
    with pytest.raises(AssertionError, match="v is on cpu"):
        api._check_same_device(q, k=torch.zeros(2, device="meta"), v=torch.zeros(2))
    import inspect
    src = inspect.getsource(api._Impl.forward) + inspect.getsource(api._Impl.backward)
    assert src.count("_check_same_device(q, ") >= 3   # k/v, eq/ek in forward; dO in backward


def test_split_scratch_stays_inside_its_budget():
    """The scratch of the split key ranges is bounded whatever the batch: with many (batch, head) pairs
    fewer tiles per pair are splittable, down to none."""
    L = _cabi.lib()
    buf = ctypes.create_string_buffer(4096)
    budget = 128 << 20
    for (B, H, Lseq, D) in [(64, 32, 2048, 128), (32, 32, 4096, 128), (8, 32, 8192, 128), (1, 32, 16384, 128),
                            (4, 8, 65536, 64), (256, 64, 2048, 16), (1, 4, 131072, 128)]:
        p = _good_params(buf)
        p.B, p.H, p.Hk, p.M, p.N, p.D = B, H, H, Lseq, Lseq, D
        p.score_mode = 1
        p.eq_stride[0], p.eq_stride[1], p.eq_stride[2] = Lseq, 0, 1
        p.ek_stride[0], p.ek_stride[1], p.ek_stride[2] = Lseq, 0, 1
        total = L.fa_workspace_bytes(ctypes.byref(p))
        plan = L.fa_workspace_plan_bytes(ctypes.byref(p))
        assert 0 < plan <= total and total - plan <= budget + 512, (B, H, Lseq, D, total - plan)
        assert L.fa_workspace_scratch_bytes(ctypes.byref(p)) == total - plan
        # a workspace of the plan's size is enough once the scratch has a home of its own
        p.workspace, p.workspace_bytes = 256 * 1024, plan
        p.eq = p.ek = p.q
        assert L.fa_validate(ctypes.byref(p), 2) == (-8 if total > plan else 0)
        p.split_scratch, p.split_scratch_bytes = 512 * 1024, total - plan
        assert L.fa_validate(ctypes.byref(p), 2) == 0
        p.split_scratch += 64
        assert L.fa_validate(ctypes.byref(p), 2) == -5
        p.split_scratch -= 64
        if total > plan:
            p.split_scratch_bytes -= 1
            assert L.fa_validate(ctypes.byref(p), 2) == -8
            p.split_scratch_bytes += 1
        p.workspace_bytes = plan - 1
        assert L.fa_validate(ctypes.byref(p), 2) == -8
    # the headline shape still splits its global-row tiles
    p = _good_params(buf)
    p.B, p.H, p.Hk, p.M, p.N, p.D, p.score_mode = 1, 32, 32, 16384, 16384, 128, 1
    p.eq_stride[2] = p.ek_stride[2] = 1
    assert L.fa_workspace_bytes(ctypes.byref(p)) - L.fa_workspace_plan_bytes(ctypes.byref(p)) > (32 << 20)


def test_drop_in_module_name():
    import flash_triton
    import flash_mi355
    assert flash_triton.attention is flash_mi355.attention
    assert flash_triton.FlashAttention is flash_mi355.FlashAttention
    assert (flash_triton.SCORE_FUNC_MODE0_NOPE, flash_triton.SCORE_FUNC_MODE1_DOC) == (0, 1)
    import inspect
    sig = inspect.signature(flash_triton.attention)
    pos = [n for n, p in sig.parameters.items() if p.kind == p.POSITIONAL_OR_KEYWORD]
    assert pos == ["q", "k", "v", "causal", "sm_scale", "eq", "ek", "score_func_mode"]   # flash_triton.py:640
    extra = {n: p for n, p in sig.parameters.items() if n not in pos}
    assert all(p.kind == p.KEYWORD_ONLY and p.default in (0, None) for p in extra.values())   # additions stay out of the way, default off
    assert [sig.parameters[n].default for n in pos][3:] == [False, None, None, None, 0]


def test_header_is_plain_c_and_matches_the_binding(tmp_path):
    """include/flash_mi355.h compiles as C (no C++ or HIP types in the boundary), a C program linked
    against the library sees the same struct size as the ctypes mirror, and validation works from C."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "flash_mi355.h"
int main(void) {
  fa_params p;
  memset(&p, 0, sizeof p);
  printf("%d %llu %llu %d %s\n", fa_version(), (unsigned long long)fa_params_size(), (unsigned long long)sizeof(fa_params),
         fa_validate(&p, 0), fa_error_string(fa_validate(&p, 0)));
  return 0;
}
''')
    exe = tmp_path / "abi"
    lib_dir = _cabi.LIB_PATH.parent
    inc = Path(__file__).resolve().parent.parent / "include"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", f"-I{inc}", str(src), "-o", str(exe), f"-L{lib_dir}",
                    "-lflash_mi355", f"-Wl,-rpath,{lib_dir}"], check=True, capture_output=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 4)
    assert int(out[0]) == _cabi.FA_ABI_VERSION
    assert int(out[1]) == int(out[2]) == ctypes.sizeof(_cabi.FaParams)
    assert int(out[3]) == -2 and "head dimension" in out[4]      # D = 0 is the first thing a zeroed struct fails
