"""GPU test of the entry point that allocates nothing: ``tlf_argmax_noalloc`` keeps its partial keys in a
file-scope device array of the library instead of a caller workspace.  It must give exactly what
``tlf_argmax`` gives, on two calls in a row that share the array, the second one smaller."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def noalloc_argmax(logits):
    from tinyllmforge_amd import _lib
    lib = _lib.load()
    out = torch.full((logits.shape[0],), -7, dtype=torch.int64, device=logits.device)
    rc = lib.tlf_argmax_noalloc(logits.data_ptr(), logits.stride(0), out.data_ptr(), logits.shape[0], logits.shape[1],
                                torch.cuda.current_stream().cuda_stream)
    return rc, out


def make_logits(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, vocab, generator=g).to(torch.bfloat16)
    top = x.float().amax(dim=1)
    for r in range(0, rows, 3):                       # planted ties: the first index must win
        idx = torch.randint(0, vocab, (3,), generator=g)
        x[r, idx] = (top[r] + 1.0).to(torch.bfloat16)
    return x


def test_noalloc_argmax_equals_argmax_on_two_calls_in_a_row():
    from oracle import ops as O
    from tinyllmforge_amd import _lib, ops as P
    lib = _lib.load()
    assert lib.tlf_argmax_noalloc_max_rows() == 1024
    big = make_logits(200, 151936, seed=1)            # 6 chunks per row
    small = make_logits(7, 5000 + 3, seed=2)          # fewer rows, 3 chunks per row, vocab % 8 != 0
    for x in (big, small):
        pad = -x.shape[1] % 8                         # rows stay 16-byte aligned: row stride 5008 for vocab 5003
        xd = torch.nn.functional.pad(x, (0, pad)).cuda()[:, :x.shape[1]]
        rc, got = noalloc_argmax(xd)
        assert rc == 0, lib.tlf_error_string(rc)
        want = P.argmax(xd)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got.cpu(), O.greedy_sample(x))
    # sizes beyond the fixed array are refused on the host, nothing is launched
    too_many = torch.zeros(1025, 64, dtype=torch.bfloat16, device="cuda")
    rc, out = noalloc_argmax(too_many)
    assert rc == -6 and b"scratch" in lib.tlf_error_string(rc)
    torch.cuda.synchronize()
    assert bool((out == -7).all())
    # the largest allowed batch, then one row again
    edge = make_logits(1024, 1024, seed=3).cuda()
    rc, got = noalloc_argmax(edge)
    assert rc == 0 and torch.equal(got, P.argmax(edge))
    rc, got = noalloc_argmax(edge[5:6])
    assert rc == 0 and torch.equal(got, P.argmax(edge[5:6]))
