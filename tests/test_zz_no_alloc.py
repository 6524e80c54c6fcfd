"""The decode attention entry point that allocates nothing
(``kllm_attn_decode_static``), called through ctypes: its partial results go to
an array the library holds on the GPU instead of a workspace.  Two calls in a
row, the second with a smaller input, must give what ``kllm_attn_decode`` gives
with a workspace of the caller's; a size beyond the array is refused."""

import ctypes
from ctypes import c_float, c_int, c_void_p

import pytest
import torch

from test_gpu_kernels import DEV, K, attention_case

pytestmark = pytest.mark.gpu


def entry_point():
    lib = ctypes.CDLL(K().library_path())
    fn = lib.kllm_attn_decode_static
    P, I = c_void_p, c_int
    fn.argtypes = [P, P, P, P, P, P, I, I, I, I, I, I, I, c_float, I, I, P, I, P]
    fn.restype = c_int
    return lib, fn


def last_error(lib):
    buf = ctypes.create_string_buffer(512)
    lib.kllm_last_error(buf, 512)
    return buf.value.decode()


def call_static(fn, c, out, nslices):
    n = c["q"].shape[0]
    return fn(c["q"].data_ptr(), out.data_ptr(), c["cache"].data_ptr(), c["pos"].data_ptr(), c["sot"].data_ptr(),
              c["bt"].data_ptr(), c["bt"].shape[1], c["ps"], n, c["H"], c["KV"], c["hd"], c["window"],
              c_float(c["scale"]), nslices, 1, None, 0, torch.cuda.current_stream().cuda_stream)


def test_two_calls_in_a_row_equal_the_entry_point_with_a_workspace():
    k_ = K()
    lib, fn = entry_point()
    cases = [attention_case(32, 4, 64, 16, torch.bfloat16, 0,
                            [(700, 1), (15, 1), (0, 1), (333, 1), (512, 1), (64, 2), (31, 1)], seed=1),
             attention_case(8, 2, 128, 16, torch.bfloat16, 37, [(200, 1), (90, 2)], seed=2)]   # smaller, second
    assert cases[1]["q"].numel() < cases[0]["q"].numel()
    for c in cases:
        n = c["q"].shape[0]
        ns = k_.attn_decode_slices(n, c["KV"], c["H"], c["hd"])
        want = torch.full_like(c["q"], float("nan"))
        part = torch.full((n * c["H"] * ns * (c["hd"] + 2),), float("nan"), device=DEV)
        k_.attn_decode(c["q"], want, part, c["cache"], c["pos"], c["sot"], c["bt"], c["ps"], c["H"], c["KV"],
                       c["hd"], c["window"], c["scale"], ns)
        got = torch.full_like(c["q"], float("nan"))
        rc = call_static(fn, c, got, ns)
        assert rc == 0, last_error(lib)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want)
        assert (got.cpu().double() - c["want"]).abs().max() < 2e-2


def test_a_size_beyond_the_array_is_refused_and_nothing_runs():
    lib, fn = entry_point()
    c = attention_case(32, 8, 128, 16, torch.bfloat16, 0, [(40, 1)] * 64, seed=3)
    out = torch.full_like(c["q"], float("nan"))
    rc = call_static(fn, c, out, 16)                     # 64 * 32 * 16 * 130 floats: four times the array
    assert rc == -2 and "exceed" in last_error(lib)
    torch.cuda.synchronize()
    assert torch.isnan(out).all()
    assert call_static(fn, c, out, 2) == 0, last_error(lib)     # and with fewer slices it fits
    torch.cuda.synchronize()
    assert (out.cpu().double() - c["want"]).abs().max() < 2e-2


def test_init_resolves_the_array_outside_any_recording():
    """The address lookup has a call of its own for callers that record graphs: after it the
    entry point does no lookup (a first call from inside a recording would be refused)."""
    lib, fn = entry_point()
    lib.kllm_attn_decode_static_init.restype = c_int
    assert lib.kllm_attn_decode_static_init() == 0, last_error(lib)
    assert lib.kllm_attn_decode_static_init() == 0
