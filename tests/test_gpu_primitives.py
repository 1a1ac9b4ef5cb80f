"""GPU parity of the two data primitives on their own (reduce, copy) against the CPU oracle.

Reference: executeReduce / executeCopy -> vector_add / vector_copy
(csrc/plugins/cuda/cuda_executor.cu:60-101, kernel/compute.h:21-102).  Bit-exact for every dtype;
sizes and offsets that are not multiples of 16 bytes are included (the reference drops such tails;
here they are processed, see the oracle header).
"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import TORCH_DTYPE, bits_equal, from_raw, mismatch_report, oracle, to_raw
from pccl_amd import _lib

pytestmark = pytest.mark.gpu


def gpu_reduce(dtype, redop, a, b, c_out):
    L = _lib.lib()
    n = a.numel()
    _lib.check(L.pccl_hip_reduce(_lib.DTYPE_ID[dtype], _lib.REDOP_ID[redop], a.data_ptr(), b.data_ptr(),
                                 c_out.data_ptr(), n, None))
    torch.cuda.synchronize()


def make(dtype, n, seed, special=False):
    g = torch.Generator().manual_seed(seed)
    if dtype == "int32":
        x = torch.randint(-2**31, 2**31 - 1, (n,), generator=g, dtype=torch.int64).to(torch.int32)
    else:
        x = (torch.randn(n, generator=g) * 3).to(TORCH_DTYPE[dtype])
        if special and n >= 16:
            vals = torch.tensor([float("inf"), float("-inf"), float("nan"), 0.0, -0.0, 65504.0, -65504.0,
                                 1e-8, -1e-8, 3.0e38, -3.0e38, 6e-5, 1e-40, 1.0, -1.0, 0.5]).to(TORCH_DTYPE[dtype])
            x[:16] = vals
    return x


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "int32"])
@pytest.mark.parametrize("redop", ["sum", "max", "min"])
@pytest.mark.parametrize("n", [1, 7, 64, 4099, 1 << 20])
def test_reduce_matches_oracle(dtype, redop, n):
    a, b = make(dtype, n, 1, special=True), make(dtype, n, 2, special=True)
    if n >= 16:
        b[:16] = a[:16].flip(0)   # inf + -inf, nan with anything, +0 with -0 ...
    want = from_raw(oracle.reduce(dtype, redop, to_raw(a), to_raw(b)), dtype)
    da, db = a.cuda(), b.cuda()
    dc = torch.empty_like(da)
    gpu_reduce(dtype, redop, da, db, dc)
    assert bits_equal(dc, want), mismatch_report(dc, want)


EDGE_F32 = [0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007FFFFF, 0x807FFFFF, 0x00800000, 0x80800000,
            0x3F800000, 0xBF800000, 0x3F800001, 0x3F7FFFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000, 0xFF800000,
            0x7F800001, 0x7FC00000, 0xFFC00000, 0x7FFFFFFF, 0xFFFFFFFF, 0x7FA00000, 0x4B800000, 0x4B7FFFFF,
            0x33800000, 0x33FFFFFF, 0x7F000000, 0xFF000000, 0x00400000, 0x80400000, 0x40490FDB, 0xC0490FDB]
EDGE_F16 = [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x83FF, 0x0400, 0x8400, 0x3C00, 0xBC00, 0x3C01, 0x3BFF,
            0x7BFF, 0xFBFF, 0x7C00, 0xFC00, 0x7C01, 0x7E00, 0xFE00, 0x7FFF, 0xFFFF, 0x7D00, 0x6400, 0x63FF,
            0x1400, 0x17FF, 0x7800, 0xF800, 0x0200, 0x8200, 0x4248, 0xC248]
EDGE_BF16 = [0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x807F, 0x0080, 0x8080, 0x3F80, 0xBF80, 0x3F81, 0x3F7F,
             0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7F81, 0x7FC0, 0xFFC0, 0x7FFF, 0xFFFF, 0x7FA0, 0x4380, 0x437F,
             0x3B80, 0x3BFF, 0x7F00, 0xFF00, 0x0040, 0x8040, 0x4049, 0xC049]


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("redop", ["sum", "max", "min"])
@pytest.mark.parametrize("lead", [0, 1])
def test_reduce_every_pair_of_edge_values(dtype, redop, lead):
    """Both zeros, the smallest and largest denormals and normals, neighbours of 1, infinities, quiet
    and signalling NaNs with several payloads, values whose sum rounds at the last place: all 1,024
    ordered pairs, bit for bit against the oracle.  `lead` = 1 shifts the operands one element off
    16-byte alignment so that the element-wise edge code runs the same pairs as the vector body."""
    codes = {"float32": EDGE_F32, "float16": EDGE_F16, "bfloat16": EDGE_BF16}[dtype]
    raw = np.uint32 if dtype == "float32" else np.uint16
    c = np.array(codes, dtype=raw)
    a = np.concatenate([np.zeros(lead, raw), np.repeat(c, len(c))])
    b = np.concatenate([np.zeros(lead, raw), np.tile(c, len(c))])
    want = oracle.reduce(dtype, redop, a[lead:].copy(), b[lead:].copy())
    ta, tb = from_raw(a, dtype).cuda(), from_raw(b, dtype).cuda()
    tc = torch.empty_like(ta)
    gpu_reduce(dtype, redop, ta[lead:], tb[lead:], tc[lead:])
    got = to_raw(tc[lead:].cpu())
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(a[lead + i])), hex(int(b[lead + i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:8]]


@pytest.mark.parametrize("dtype", ["float8_e4m3", "float8_e5m2"])
@pytest.mark.parametrize("redop", ["sum", "max", "min"])
def test_fp8_reduce_all_operand_pairs(dtype, redop):
    """Reference vec.h:272-426 (widen to f16, add, narrow with saturation): every one of the 65,536
    operand pairs, laid out so that vector bodies, heads and tails all occur (offset 3, odd length)."""
    codes = torch.arange(256, dtype=torch.int16).to(torch.uint8)
    a = torch.cat([torch.zeros(3, dtype=torch.uint8), codes.repeat_interleave(256)])
    b = torch.cat([torch.zeros(3, dtype=torch.uint8), codes.repeat(256)])
    want = torch.from_numpy(oracle.reduce(dtype, redop, a.numpy().copy(), b.numpy().copy()))
    da, db = a.cuda(), b.cuda()
    dc = torch.empty_like(da)
    gpu_reduce(dtype, redop, da[3:], db[3:], dc[3:])
    got = dc[3:].cpu()
    bad = (got != want[3:]).nonzero().flatten()
    assert bad.numel() == 0, [(hex(int(a[3 + i])), hex(int(b[3 + i])), hex(int(got[i])), hex(int(want[3 + i]))) for i in bad[:8]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shift", [(0, 0, 0), (1, 1, 1), (3, 3, 3), (1, 2, 3), (0, 1, 0)])
def test_reduce_unaligned_offsets(dtype, shift):
    """Element offsets that break 16-byte alignment, equal and unequal between the operands."""
    n = 10007
    a, b = make(dtype, n + 8, 3), make(dtype, n + 8, 4)
    sa, sb, sc = shift
    want = from_raw(oracle.reduce(dtype, "sum", to_raw(a[sa:sa + n]), to_raw(b[sb:sb + n])), dtype)
    da, db = a.cuda(), b.cuda()
    dc = torch.zeros(n + 8, dtype=TORCH_DTYPE[dtype], device="cuda")
    gpu_reduce(dtype, "sum", da[sa:sa + n], db[sb:sb + n], dc[sc:sc + n])
    assert bits_equal(dc[sc:sc + n], want), mismatch_report(dc[sc:sc + n], want)
    assert torch.all(dc[:sc] == 0) and torch.all(dc[sc + n:] == 0), "wrote outside the range"


def test_reduce_in_place_aliasing():
    """c aliases b, as every schedule of the reference uses it (off1 == off2)."""
    n = 1 << 16
    a, b = make("bfloat16", n, 5), make("bfloat16", n, 6)
    want = from_raw(oracle.reduce("bfloat16", "sum", to_raw(a), to_raw(b)), "bfloat16")
    da, db = a.cuda(), b.cuda()
    gpu_reduce("bfloat16", "sum", da, db, db)
    assert bits_equal(db, want)


@pytest.mark.parametrize("nbytes", [1, 15, 16, 17, 4096, 65537, 1 << 22])
@pytest.mark.parametrize("shift", [(0, 0), (1, 1), (5, 5), (1, 2)])
def test_copy_bytes(nbytes, shift):
    L = _lib.lib()
    src = torch.randint(0, 256, (nbytes + 16,), dtype=torch.uint8)
    dsrc = src.cuda()
    ddst = torch.zeros(nbytes + 16, dtype=torch.uint8, device="cuda")
    s, d = shift
    _lib.check(L.pccl_hip_copy(_lib.DTYPE_ID["float8_e4m3"], dsrc[s:].data_ptr(), ddst[d:].data_ptr(), nbytes, None))
    torch.cuda.synchronize()
    out = ddst.cpu()
    assert torch.equal(out[d:d + nbytes], src[s:s + nbytes])
    assert torch.all(out[:d] == 0) and torch.all(out[d + nbytes:] == 0)


def test_bad_arguments_are_errors():
    L = _lib.lib()
    x = torch.zeros(16, device="cuda")
    assert L.pccl_hip_reduce(17, 0, x.data_ptr(), x.data_ptr(), x.data_ptr(), 4, None) == _lib.ERR_UNSUPPORTED   # no such dtype
    assert L.pccl_hip_reduce(0, 9, x.data_ptr(), x.data_ptr(), x.data_ptr(), 4, None) == _lib.ERR_INVALID
    assert L.pccl_hip_reduce(0, 0, None, x.data_ptr(), x.data_ptr(), 4, None) == _lib.ERR_INVALID
    assert b"null" in L.pccl_hip_last_error()
