"""The allocation-free column sum (tf_colsum_noalloc) through the C ABI: equal, bit for bit, to
tf_colsum on the same input, on two calls in a row of which the second is smaller (the library's
fixed scratch array then still holds the first call's partial sums), for fp16 and bf16 input and
fp32 output; sizes beyond the fixed scratch are refused.  Collected last: the file name sorts after
every other test file."""
import pytest
import torch

from tritonformer_amd import _lib

pytestmark = pytest.mark.gpu


def colsum(lib, x, out_dtype, noalloc):
    rows, cols = x.shape
    out = torch.full((cols,), float("nan"), dtype=out_dtype, device=x.device)
    stream = torch.cuda.current_stream().cuda_stream
    code, ocode = _lib.dtype_code(x.dtype), _lib.dtype_code(out_dtype)
    if noalloc:
        rc = lib.tf_colsum_noalloc(stream, code, ocode, rows, cols, x.data_ptr(), x.stride(0), out.data_ptr())
    else:
        nbytes = lib.tf_colsum_partial_bytes(rows, cols)
        part = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        rc = lib.tf_colsum(stream, code, ocode, rows, cols, x.data_ptr(), x.stride(0), out.data_ptr(),
                           part.data_ptr(), nbytes)
    _lib.check(rc)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype,out_dtype", [(torch.float16, torch.float16), (torch.bfloat16, torch.float32)])
def test_noalloc_colsum_equals_colsum_on_two_calls_in_a_row(dtype, out_dtype, dev):
    lib = _lib.load()
    g = torch.Generator().manual_seed(3)
    big = torch.randn(8192, 3072, generator=g).to(dtype).to(dev)
    small = torch.randn(77, 333, generator=g).to(dtype).to(dev)      # ragged: element-wise load path
    for x in (big, small, big[:4096, :1024]):                       # second and third calls are smaller
        got = colsum(lib, x, out_dtype, noalloc=True)
        want = colsum(lib, x, out_dtype, noalloc=False)
        assert torch.equal(got, want)
        ref = x.double().sum(0)
        tol = 2e-3 if out_dtype != torch.float32 else 1e-5
        assert ((got.double() - ref).norm() / ref.norm()).item() < tol


def test_noalloc_colsum_refuses_what_its_scratch_cannot_hold(dev):
    lib = _lib.load()
    limit = lib.tf_colsum_noalloc_max_partial_bytes()
    assert limit == 4 << 20
    rows, cols = 8, 1 << 21                       # one group x 2M columns of fp32 partial sums = 8 MiB
    assert lib.tf_colsum_partial_bytes(rows, cols) > limit
    x = torch.zeros(8, 8, dtype=torch.float16, device=dev)           # never read: the check comes first
    out = torch.zeros(cols, dtype=torch.float16, device=dev)
    assert lib.tf_colsum_noalloc(None, 0, 0, rows, cols, x.data_ptr(), cols, out.data_ptr()) == -5
    assert lib.tf_colsum_noalloc(None, 0, 0, 16, 64, None, 64, out.data_ptr()) == -1
    assert lib.tf_colsum_noalloc(None, 2, 2, 16, 64, x.data_ptr(), 64, out.data_ptr()) == -2
