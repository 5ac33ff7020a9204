"""CPU oracle: grouped GEMM.  Test infrastructure only.

The reference calls the un-vendored package ``grouped_gemm==0.3.0`` (setup.py:71-73)
through megablocks/grouped_gemm_util.py:25-26.  Its arithmetic is fixed by the call
sites (megablocks/layers/mlp.py:414-491,521-523, megablocks/layers/glu.py:84-205) and by
the reference tests that equate it with dense matmul (tests/layers/glu_test.py:64-102,
tests/layers/dmoe_test.py:216-241): for consecutive row groups r_e of ``batch_sizes[e]``
rows,
    default  out[r_e] = a[r_e] @ b[e]
    trans_b  out[r_e] = a[r_e] @ b[e].T
    trans_a  out[e]   = a[r_e].T @ b[r_e]      (zero matrix for an empty group)
with fp32 accumulation and the result stored in the input dtype.
"""
import torch


def gmm(a, b, batch_sizes, trans_a=False, trans_b=False, c=None):
    sizes = [int(v) for v in batch_sizes]
    assert a.ndim == 2 and sum(sizes) == a.shape[0]
    if trans_a:
        assert b.ndim == 2 and b.shape[0] == a.shape[0] and not trans_b
        out = torch.zeros((len(sizes), a.shape[1], b.shape[1]), dtype=torch.float32)
        start = 0
        for e, n in enumerate(sizes):
            if n:
                out[e] = a[start:start + n].float().t() @ b[start:start + n].float()
            start += n
    else:
        assert b.ndim == 3 and b.shape[0] == len(sizes)
        cols = b.shape[1] if trans_b else b.shape[2]
        out = torch.zeros((a.shape[0], cols), dtype=torch.float32)
        start = 0
        for e, n in enumerate(sizes):
            if n:
                be = b[e].float()
                out[start:start + n] = a[start:start + n].float() @ (be.t() if trans_b else be)
            start += n
    out = out.to(a.dtype)
    if c is not None:
        c.copy_(out)
        return c
    return out
