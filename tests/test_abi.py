"""The C-ABI library loads without a GPU, exports every symbol include/fwa2.h
declares, and rejects contract violations before touching a device."""
import ctypes
import os
import re

import pytest

from flash_window_attention_v2_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_abi.lib_path()):
        import __graft_entry__

        __graft_entry__.build()
    return _abi.load()


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "fwa2.h")).read()
    declared = set(re.findall(r"^\s*(?:int|size_t|void|const char\*)\s+(fwa2_\w+)\s*\(", header, flags=re.M))
    assert declared == set(_abi.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.fwa2_abi_version() == _abi.ABI_VERSION


def test_struct_layout_matches(lib):
    # a problem of the wrong size is refused, one of the right size gets past the layout check
    p = _abi.new_problem()
    p.struct_bytes -= 8
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT
    assert b"layout mismatch" in lib.fwa2_last_error()
    p = _abi.new_problem()
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT
    assert b"layout" not in lib.fwa2_last_error()


def _good_problem(n=64, bw=8, heads=2, backward=False):
    p = _abi.new_problem()
    p.dtype, p.mask_dtype, p.scale_kind = _abi.BF16, _abi.BF16, _abi.SCALE_DEFAULT
    p.bw, p.heads, p.n, p.head_dim, p.n_windows = bw, heads, n, 32, 1
    fake = 0x10000  # never dereferenced by fwa2_validate
    t4 = lambda: _abi.Tensor4(fake, heads * n * 32, n * 32, 32)
    p.q, p.k, p.v, p.o = t4(), t4(), t4(), t4()
    p.lse, p.lse_stride_bw, p.lse_stride_h = fake, heads * n, n
    if backward:
        p.d_o, p.dq, p.dk, p.dv = t4(), t4(), t4(), t4()
        p.workspace, p.workspace_bytes = 0x100000, 1 << 30
    return p


def test_validate_accepts_and_rejects(lib):
    assert lib.fwa2_validate(_good_problem(), 0) == _abi.OK
    assert lib.fwa2_validate(_good_problem(backward=True), 1) == _abi.OK

    p = _good_problem()
    p.dtype = _abi.F32
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT and b"fp16 and bf16" in lib.fwa2_last_error()

    p = _good_problem()
    p.head_dim = 256
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT and b"up to 128" in lib.fwa2_last_error()

    p = _good_problem()
    p.head_dim = 20     # rows are read in 16-byte chunks
    assert lib.fwa2_validate(p, 0) == _abi.ERR_UNSUPPORTED and b"multiples of 8" in lib.fwa2_last_error()
    for hd in (8, 16, 24, 32):
        p.head_dim = hd
        assert lib.fwa2_validate(p, 0) == _abi.OK
    p.head_dim = 64     # the row stride of _good_problem is 32
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT and b"overlaps rows" in lib.fwa2_last_error()

    p = _good_problem()
    p.n_keys = 96       # more keys than queries: legal, bias / mask rows must then hold 96 entries
    assert lib.fwa2_validate(p, 0) == _abi.OK
    p.bias = _abi.Tensor3(0x10000, 64 * 64, 64)
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT and b"number of keys" in lib.fwa2_last_error()
    p.bias = _abi.Tensor3(0x10000, 64 * 96, 96)
    assert lib.fwa2_validate(p, 0) == _abi.OK
    p.grid_h, p.grid_w, p.win_h, p.win_w = 16, 16, 8, 8     # a window map needs keys == queries
    p.bw = 8
    assert lib.fwa2_validate(p, 0) == _abi.ERR_UNSUPPORTED and b"window map" in lib.fwa2_last_error()
    p = _good_problem()
    p.scale_head_dim = 20       # rows of 20 elements padded with zeros to 32: legal
    assert lib.fwa2_validate(p, 0) == _abi.OK
    p.scale_head_dim = 40       # more than the rows hold
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT and b"scale_head_dim" in lib.fwa2_last_error()

    p = _good_problem()
    p.q = _abi.Tensor4(0x10002, 4096, 2048, 32)  # rows not 16-byte aligned
    assert lib.fwa2_validate(p, 0) == _abi.ERR_UNSUPPORTED

    p = _good_problem()
    big = 1 << 24       # rows are addressed with a 24-bit multiply and a 32-bit byte offset inside a unit
    p.q = _abi.Tensor4(0x10000, 2 * 64 * big, 64 * big, big)
    assert lib.fwa2_validate(p, 0) == _abi.ERR_UNSUPPORTED and b"2^24" in lib.fwa2_last_error()
    p = _good_problem(n=1 << 16)
    wide = 1 << 14      # 2^16 rows of 2^14 elements: 2^31 bytes in one unit
    p.q = _abi.Tensor4(0x10000, 2 * (1 << 16) * wide, (1 << 16) * wide, wide)
    assert lib.fwa2_validate(p, 0) == _abi.ERR_UNSUPPORTED and b"2^31 bytes" in lib.fwa2_last_error()

    p = _good_problem()
    p.scale_kind = _abi.SCALE_TENSOR  # without a pointer
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT

    p = _good_problem(bw=9)
    p.mask = _abi.Tensor3(0x10000, 64 * 64, 64)
    p.n_windows = 4  # 9 % 4 != 0
    assert lib.fwa2_validate(p, 0) == _abi.ERR_INVALID_ARGUMENT and b"multiple of n_windows" in lib.fwa2_last_error()

    p = _good_problem(backward=True)
    p.bias = _abi.Tensor3(0x10000, 64 * 64, 64)  # bias without dbias / workspace
    assert lib.fwa2_validate(p, 1) == _abi.ERR_INVALID_ARGUMENT


def test_validate_survives_arbitrary_descriptions(lib):
    """Seeded random problem descriptions (sizes from zero to absurd, negative strides, odd pointers, window maps
    that do not divide the grid): fwa2_validate and the workspace query only ever answer with a status or a size,
    on a machine without a GPU too, and a rejected description always leaves a message."""
    import random
    rng = random.Random(20240607)
    sizes = [-3, 0, 1, 2, 7, 8, 31, 32, 63, 64, 100, 144, 196, 256, 257, 576, 1024, 1025, 4096, 1 << 20, (1 << 31) - 1]
    strides = [-64, 0, 1, 8, 31, 32, 40, 64, 2048, 4096, 1 << 20, 1 << 24, 1 << 40, (1 << 62)]
    ptrs = [0, 0x10000, 0x10002, 0x10008, 0x7fff00000010]
    seen = set()
    for _ in range(4000):
        backward = rng.random() < 0.5
        p = _good_problem(n=rng.choice([64, 144, 256, 576]), bw=rng.choice([1, 8, 64]), heads=rng.choice([1, 3]),
                          backward=backward)
        for _ in range(rng.randint(1, 4)):
            what = rng.randrange(12)
            if what == 0: p.n = rng.choice(sizes)
            elif what == 1: p.bw = rng.choice(sizes)
            elif what == 2: p.heads = rng.choice(sizes)
            elif what == 3: p.head_dim = rng.choice(sizes)
            elif what == 4: p.n_keys = rng.choice(sizes)
            elif what == 5: p.n_windows = rng.choice(sizes)
            elif what == 6:
                t = rng.choice([p.q, p.k, p.v, p.o, p.d_o, p.dq, p.dk, p.dv])
                t.ptr, t.stride_bw, t.stride_h, t.stride_n = (rng.choice(ptrs), rng.choice(strides), rng.choice(strides),
                                                               rng.choice(strides))
            elif what == 7:
                t = rng.choice([p.bias, p.mask])
                t.ptr, t.stride_a, t.stride_n = rng.choice(ptrs), rng.choice(strides), rng.choice(strides)
            elif what == 8:
                p.grid_h, p.grid_w, p.win_h, p.win_w, p.shift_h, p.shift_w = (rng.choice(sizes[:12]) for _ in range(6))
            elif what == 9: p.dtype, p.mask_dtype = rng.randrange(-1, 5), rng.randrange(-1, 5)
            elif what == 10: p.scale_kind, p.scale_head_dim = rng.randrange(-1, 4), rng.choice(sizes[:10])
            else: p.lse_stride_bw, p.lse_stride_h, p.workspace_bytes = rng.choice(strides), rng.choice(strides), rng.choice(sizes)
        st = lib.fwa2_validate(p, int(backward))
        assert st in (_abi.OK, _abi.ERR_INVALID_ARGUMENT, _abi.ERR_UNSUPPORTED), st
        if st != _abi.OK:
            assert len(lib.fwa2_last_error()) > 0
        need = lib.fwa2_backward_workspace_bytes(p)
        assert 0 <= need < (1 << 62) or need == (1 << 64) - 1        # a size, or "no device can hold this"
        seen.add(st)
    assert seen == {_abi.OK, _abi.ERR_INVALID_ARGUMENT, _abi.ERR_UNSUPPORTED}


def test_workspace_size_is_reported(lib):
    p = _good_problem(n=256, bw=4096, heads=3, backward=True)
    p.bias = _abi.Tensor3(0x10000, 65536, 256)
    need = lib.fwa2_backward_workspace_bytes(p)
    # one fp32 [256, 256] partial per persistent workgroup plus the transposed bias
    assert 3 * 256 * 256 * 4 < need < 512 * 1024 * 1024
    p.workspace, p.workspace_bytes, p.dbias = 0x100000, need - 1, 0x20000
    assert lib.fwa2_validate(p, 1) == _abi.ERR_INVALID_ARGUMENT and b"workspace" in lib.fwa2_last_error()
    p.workspace_bytes = need
    assert lib.fwa2_validate(p, 1) == _abi.OK


def test_status_to_exception(lib):
    p = _good_problem()
    p.head_dim = 20
    with pytest.raises(NotImplementedError):
        _abi.check(lib.fwa2_validate(p, 0), "validate")
    p.head_dim = 200
    with pytest.raises(AssertionError):
        _abi.check(lib.fwa2_validate(p, 0), "validate")


def test_function_rejects_bad_arguments_on_cpu():
    """The reference asserts before launching (attn_kernel_forward.py:265-292);
    so does this Function, which lets the checks run without a GPU."""
    import torch

    from flash_window_attention_v2_amd import flash_win_attn_v2_func

    q = torch.randn(4, 2, 64, 32, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):            # CPU tensors
        flash_win_attn_v2_func(q, q, q)
    with pytest.raises(AssertionError):            # fp32 inputs
        flash_win_attn_v2_func(q.float(), q.float(), q.float())
    with pytest.raises(AssertionError):            # mixed dtypes
        flash_win_attn_v2_func(q, q.half(), q)
    with pytest.raises(AssertionError):            # logit_scale must be a tensor
        flash_win_attn_v2_func(q, q, q, 1.0)


def test_header_compiles_as_c_and_cxx(tmp_path):
    """include/fwa2.h is the boundary a C or C++ host binds: it must be self-contained in both languages
    and lay the problem struct out exactly as the ctypes mirror does."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None or shutil.which("g++") is None:
        pytest.skip("no host compiler")
    src = tmp_path / "use_header.c"
    src.write_text(
        '#include "fwa2.h"\n#include <stdio.h>\n'
        'int main(void) { fwa2_problem p; (void)p; printf("%zu %zu %zu\\n", sizeof(fwa2_problem), '
        'sizeof(fwa2_tensor4), sizeof(fwa2_tensor3)); return 0; }\n')
    inc = os.path.join(ROOT, "include")
    exe = tmp_path / "use_header"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", inc, str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert [int(x) for x in out] == [ctypes.sizeof(_abi.Problem), ctypes.sizeof(_abi.Tensor4), ctypes.sizeof(_abi.Tensor3)]
    cxx = tmp_path / "use_header.cpp"
    cxx.write_text('#include "fwa2.h"\nint main() { fwa2_problem p{}; return p.n; }\n')
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-I", inc, "-fsyntax-only", str(cxx)], check=True)


def test_static_scratch_backward_refuses_oversize_without_a_device(lib):
    """The allocation-free backward sizes the problem before it looks for a device: windows of 576 tokens need
    more scratch than the library's static buffer and are refused with the limit in the message."""
    p = _good_problem(n=576, bw=256, heads=6, backward=True)
    p.bias.ptr, p.bias.stride_a, p.bias.stride_n = 0x10000, 576 * 576, 576
    p.dbias = 0x10000
    assert lib.fwa2_backward_workspace_bytes(p) > _abi.STATIC_SCRATCH_BYTES
    assert lib.fwa2_backward_static(p) == _abi.ERR_UNSUPPORTED
    msg = lib.fwa2_last_error().decode()
    assert "static buffer holds" in msg and str(_abi.STATIC_SCRATCH_BYTES) in msg
    header = open(os.path.join(ROOT, "include", "fwa2.h")).read()
    assert re.search(r"#define FWA2_STATIC_SCRATCH_BYTES \(\(size_t\)128 << 20\)", header) and _abi.STATIC_SCRATCH_BYTES == 128 << 20


def test_problem_filled_the_way_a_binding_fills_it(lib):
    """A struct built by keyword, as a ctypes binding of the reference's forward call site would build it
    (flash_win_attn_v2/flash_window_attention_v2.py:22-24), passes validation with the version the library
    reports and is refused with any other."""
    bw, h, n, d, nw = 8, 3, 64, 32, 4
    t4 = lambda: _abi.Tensor4(0x10000, h * n * d, n * d, d)
    t3 = lambda: _abi.Tensor3(0x10000, n * n, n)
    fields = dict(struct_bytes=ctypes.sizeof(_abi.Problem), dtype=_abi.BF16, mask_dtype=_abi.BF16,
                  scale_kind=_abi.SCALE_TENSOR, bw=bw, heads=h, n=n, head_dim=d, n_windows=nw,
                  q=t4(), k=t4(), v=t4(), o=t4(), logit_scale=0x10000, bias=t3(), mask=t3(), lse=0x10000,
                  lse_stride_bw=h * n, lse_stride_h=n, stream=None)
    p = _abi.Problem(abi_version=lib.fwa2_abi_version(), **fields)
    assert lib.fwa2_abi_version() == 4
    assert lib.fwa2_validate(ctypes.byref(p), 0) == _abi.OK, lib.fwa2_last_error()
    p = _abi.Problem(abi_version=1, **fields)
    assert lib.fwa2_validate(ctypes.byref(p), 0) == _abi.ERR_INVALID_ARGUMENT
    assert b"abi 1, library 480 bytes / abi 4" in lib.fwa2_last_error()
