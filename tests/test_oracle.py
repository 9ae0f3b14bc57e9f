"""Pins the CPU oracle (oracle/clusten_oracle.py): the gather expressions restated from the reference's
kernel test scripts are checked against independent statements of the same sums and against what the
mathematics fixes.  The reference holds no golden vectors for these ops, so none are used.

Each check is chosen so that a plausible mistake fails it: a transposed operand (dense matmul case),
a wrong gather axis or index expansion (one-hot / identity cases, integer-exact case), a dropped head
or batch offset (slice independence), a mis-ordered (ic, c) output (WF layout case), a mis-indexed
gradient (random upstream gradients, index_add_ formulation, conservation law, gradcheck).
"""
import numpy as np
import pytest
import torch

from oracle import build as cref
from oracle import clusten_oracle as oracle


def _tiny(seed=0, b=2, h=2, n=7, c=3, m=4, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, n, c, generator=g, dtype=dtype)
    k = torch.randn(b, h, n, c, generator=g, dtype=dtype)
    v = torch.randn(b, h, n, c, generator=g, dtype=dtype)
    a = torch.randn(b, h, n, m, generator=g, dtype=dtype)
    idx = torch.randint(n, (b, n, m), generator=g)  # duplicates allowed, like the reference scripts
    return q, k, v, a, idx


def _tiny_wf(seed=0, b=2, n=9, n_=4, c=5, m=4, ic=3, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(b, n_, m, ic, generator=g, dtype=dtype)
    f = torch.randn(b, n, c, generator=g, dtype=dtype)
    idx = torch.randint(n, (b, n_, m), generator=g)
    return w, f, idx


# ---- forward vs. nested loops (numpy float64) and vs. the C loops ---------------------------------

@pytest.mark.parametrize("seed", [0, 1, 2])
def test_forward_matches_nested_loops(seed):
    q, k, v, a, idx = _tiny(seed)
    np.testing.assert_allclose(oracle.qk_gather(q, k, idx).numpy(), oracle.qk_loops(q, k, idx), rtol=0, atol=1e-13)
    np.testing.assert_allclose(oracle.av_gather(a, v, idx).numpy(), oracle.av_loops(a, v, idx), rtol=0, atol=1e-13)
    w, f, widx = _tiny_wf(seed)
    np.testing.assert_allclose(oracle.wf_gather(w, f, widx).numpy(), oracle.wf_loops(w, f, widx), rtol=0, atol=1e-13)


def test_forward_matches_c_loops_reference_script_shapes():
    # shapes of clusten/test_qk_kernel.py:14-18 and test_wf_kernel.py:14-19 with a smaller batch
    g = torch.Generator().manual_seed(7)
    b, h, n, m, c = 4, 4, 196, 48, 32
    q, k, v = (torch.randn(b, h, n, c, generator=g) for _ in range(3))
    a = torch.randn(b, h, n, m, generator=g)
    idx = torch.randint(n, (b, n, m), generator=g)
    assert oracle.rel_err(oracle.qk_gather(q, k, idx), cref.qk_forward(q, k, idx)) < 2e-6
    assert oracle.rel_err(oracle.av_gather(a, v, idx), cref.av_forward(a, v, idx)) < 2e-6
    n_, ic = 64, 4
    w = torch.randn(b, n_, m, ic, generator=g)
    f = torch.randn(b, n, c, generator=g)
    widx = torch.randint(n, (b, n_, m), generator=g)
    assert oracle.rel_err(oracle.wf_gather(w, f, widx), cref.wf_forward(w, f, widx)) < 2e-6


def test_backward_matches_nested_loops_and_c_loops():
    q, k, v, a, idx = _tiny(3)
    g_attn = torch.randn_like(a)
    g_feat = torch.randn_like(q)
    dq, dk = oracle.qk_gather_backward(g_attn, q, k, idx)
    dq_l, dk_l = oracle.qk_backward_loops(g_attn, q, k, idx)
    np.testing.assert_allclose(dq.numpy(), dq_l, atol=1e-13)
    np.testing.assert_allclose(dk.numpy(), dk_l, atol=1e-13)
    da, dv = oracle.av_gather_backward(g_feat, a, v, idx)
    da_l, dv_l = oracle.av_backward_loops(g_feat, a, v, idx)
    np.testing.assert_allclose(da.numpy(), da_l, atol=1e-13)
    np.testing.assert_allclose(dv.numpy(), dv_l, atol=1e-13)
    w, f, widx = _tiny_wf(3)
    g_out = torch.randn(w.shape[0], w.shape[1], w.shape[3], f.shape[2], dtype=torch.float64)
    dw, df = oracle.wf_gather_backward(g_out, w, f, widx)
    dw_l, df_l = oracle.wf_backward_loops(g_out, w, f, widx)
    np.testing.assert_allclose(dw.numpy(), dw_l, atol=1e-13)
    np.testing.assert_allclose(df.numpy(), df_l, atol=1e-13)
    # C loops, float32 in / double accumulate
    for x, y in zip(cref.qk_backward(g_attn, q, k, idx), (dq, dk)):
        assert oracle.rel_err(x, y) < 1e-6
    for x, y in zip(cref.av_backward(g_feat, a, v, idx), (da, dv)):
        assert oracle.rel_err(x, y) < 1e-6
    for x, y in zip(cref.wf_backward(g_out, w, f, widx), (dw, df)):
        assert oracle.rel_err(x, y) < 1e-6


# ---- special cases that reduce to library routines --------------------------------------------------

def test_dense_lists_reduce_to_matmul():
    # idx[b,i,:] = arange(n): QK = q @ k^T, AV = attn @ v, WF = w^T @ feat (the model's global-attention branch)
    g = torch.Generator().manual_seed(11)
    b, h, n, c = 2, 3, 10, 4
    q, k, v = (torch.randn(b, h, n, c, generator=g, dtype=torch.float64) for _ in range(3))
    idx = torch.arange(n).expand(b, n, n).contiguous()
    torch.testing.assert_close(oracle.qk_gather(q, k, idx), q @ k.transpose(-1, -2), rtol=0, atol=1e-13)
    a = torch.randn(b, h, n, n, generator=g, dtype=torch.float64)
    torch.testing.assert_close(oracle.av_gather(a, v, idx), a @ v, rtol=0, atol=1e-13)
    n_, ic = 6, 3
    w = torch.randn(b, n_, n, ic, generator=g, dtype=torch.float64)
    f = torch.randn(b, n, c, generator=g, dtype=torch.float64)
    widx = torch.arange(n).expand(b, n_, n).contiguous()
    torch.testing.assert_close(oracle.wf_gather(w, f, widx), torch.einsum("bimk,bmc->bikc", w, f), rtol=0, atol=1e-13)


def test_identity_list_is_rowwise_dot():
    q, k, _, _, _ = _tiny(5, m=1)
    b, h, n, c = q.shape
    idx = torch.arange(n).reshape(1, n, 1).expand(b, n, 1).contiguous()
    torch.testing.assert_close(oracle.qk_gather(q, k, idx)[..., 0], (q * k).sum(-1), rtol=0, atol=1e-13)


def test_one_hot_weights_are_a_pure_gather_bit_exact():
    # one-hot attn / weights select one neighbour: result must equal torch's own gather bit for bit
    g = torch.Generator().manual_seed(13)
    b, h, n, c, m = 2, 2, 12, 5, 6
    v = torch.randn(b, h, n, c, generator=g)
    idx = torch.randint(n, (b, n, m), generator=g)
    pick = torch.randint(m, (b, h, n), generator=g)
    a = torch.nn.functional.one_hot(pick, m).to(torch.float32)
    chosen = idx.unsqueeze(1).expand(b, h, n, m).gather(3, pick.unsqueeze(-1))           # (b,h,n,1)
    expect = v.gather(2, chosen.expand(-1, -1, -1, c))
    assert torch.equal(oracle.av_gather(a, v, idx), expect)
    n_, ic = 5, 2
    f = torch.randn(b, n, c, generator=g)
    widx = torch.randint(n, (b, n_, m), generator=g)
    wpick = torch.randint(m, (b, n_, ic), generator=g)
    w = torch.nn.functional.one_hot(wpick, m).to(torch.float32).permute(0, 1, 3, 2).contiguous()  # (b,n_,m,ic)
    rows = widx.gather(2, wpick)                                                           # (b,n_,ic)
    expect = f.gather(1, rows.reshape(b, -1, 1).expand(-1, -1, c)).reshape(b, n_, ic, c)
    assert torch.equal(oracle.wf_gather(w, f, widx), expect)


def test_integer_valued_data_is_exact():
    # small integers: every fp32 product and partial sum is exact, so index handling must be bit exact
    g = torch.Generator().manual_seed(17)
    b, h, n, c, m = 2, 2, 20, 8, 7
    q = torch.randint(-8, 9, (b, h, n, c), generator=g).float()
    k = torch.randint(-8, 9, (b, h, n, c), generator=g).float()
    idx = torch.randint(n, (b, n, m), generator=g)
    expect = torch.from_numpy(oracle.qk_loops(q, k, idx)).float()
    assert torch.equal(oracle.qk_gather(q, k, idx), expect)
    assert torch.equal(cref.qk_forward(q, k, idx), expect)


def test_uniform_weights_give_neighbourhood_mean():
    _, _, v, _, idx = _tiny(19)
    b, h, n, c = v.shape
    m = idx.shape[-1]
    a = torch.full((b, h, n, m), 1.0 / m, dtype=v.dtype)
    expect = torch.stack([torch.stack([v[bi, :, idx[bi, i]].mean(dim=1) for i in range(n)], dim=1) for bi in range(b)])
    torch.testing.assert_close(oracle.av_gather(a, v, idx), expect, rtol=0, atol=1e-13)


# ---- invariants --------------------------------------------------------------------------------------

def test_slot_permutation_invariants():
    q, k, v, a, idx = _tiny(23)
    perm = torch.randperm(idx.shape[-1], generator=torch.Generator().manual_seed(1))
    torch.testing.assert_close(oracle.qk_gather(q, k, idx[..., perm]), oracle.qk_gather(q, k, idx)[..., perm])
    torch.testing.assert_close(oracle.av_gather(a[..., perm], v, idx[..., perm]), oracle.av_gather(a, v, idx),
                               rtol=0, atol=1e-13)


def test_batch_and_head_slices_are_independent():
    q, k, v, a, idx = _tiny(29)
    full = oracle.qk_gather(q, k, idx)
    torch.testing.assert_close(oracle.qk_gather(q[1:2, 1:2], k[1:2, 1:2], idx[1:2]), full[1:2, 1:2])
    full = oracle.av_gather(a, v, idx)
    torch.testing.assert_close(oracle.av_gather(a[1:2, 0:1], v[1:2, 0:1], idx[1:2]), full[1:2, 0:1])


def test_duplicates_contribute_twice_and_linearity():
    _, _, v, a, idx = _tiny(31)
    idx2 = idx.clone()
    idx2[..., 1] = idx2[..., 0]  # slot 1 repeats slot 0
    a_merged = a.clone()
    a_merged[..., 0] += a_merged[..., 1]
    a_merged[..., 1] = 0
    torch.testing.assert_close(oracle.av_gather(a, v, idx2), oracle.av_gather(a_merged, v, idx2), rtol=0, atol=1e-13)
    torch.testing.assert_close(oracle.av_gather(2 * a, v, idx) + oracle.av_gather(a, 3 * v, idx),
                               5 * oracle.av_gather(a, v, idx), rtol=0, atol=1e-12)


def test_wf_output_order_is_ic_then_channel():
    # reshape(b, n_, ic*c) must put inner channel ic at columns [ic*c, (ic+1)*c) (aff_transformer.py:361)
    w, f, idx = _tiny_wf(37)
    out = oracle.wf_gather(w, f, idx)
    b, n_, ic, c = out.shape
    for i in range(ic):
        single = oracle.wf_gather(w[..., i:i + 1], f, idx)[:, :, 0]
        torch.testing.assert_close(out.reshape(b, n_, ic * c)[:, :, i * c:(i + 1) * c], single)


def test_chunked_equals_unchunked():
    q, k, v, a, idx = _tiny(41, b=5)
    assert torch.equal(oracle.qk_gather_chunked(q, k, idx, 2), oracle.qk_gather(q, k, idx))
    assert torch.equal(oracle.av_gather_chunked(a, v, idx, 2), oracle.av_gather(a, v, idx))


# ---- backward: what the mathematics fixes -------------------------------------------------------------

def test_gradcheck_float64():
    q, k, v, a, idx = _tiny(43, b=1, h=2, n=5, c=3, m=3)
    for t in (q, k, v, a):
        t.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda x, y: oracle.qk_gather(x, y, idx), (q, k))
    assert torch.autograd.gradcheck(lambda x, y: oracle.av_gather(x, y, idx), (a, v))
    w, f, widx = _tiny_wf(43, b=1, n=5, n_=3, c=2, m=3, ic=2)
    w.requires_grad_(True)
    f.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda x, y: oracle.wf_gather(x, y, widx), (w, f))


def test_scatter_gradient_is_index_add_and_conserves_mass():
    q, k, _, a, idx = _tiny(47)
    b, h, n, c = q.shape
    m = idx.shape[-1]
    g = torch.randn_like(a)
    _, dk = oracle.qk_gather_backward(g, q, k, idx)
    # d_key as an explicit index_add_ of the outer products q[i] * g[i,j]
    expect = torch.zeros_like(k)
    for bi in range(b):
        contrib = (g[bi].unsqueeze(-1) * q[bi].unsqueeze(2)).reshape(h, n * m, c)        # (h, n*m, c)
        expect[bi].index_add_(1, idx[bi].reshape(-1), contrib)
    torch.testing.assert_close(dk, expect, rtol=0, atol=1e-12)
    # sum over destination rows = sum over all (i,j) products, whatever the indices are
    torch.testing.assert_close(dk.sum(2), (g.sum(-1, keepdim=True) * q).sum(2), rtol=0, atol=1e-12)


def test_rel_err_metric():
    x = torch.tensor([1.0, 2.0, 4.0], dtype=torch.float64)
    assert oracle.rel_err(x, x) == 0.0
    assert abs(oracle.rel_err(x + torch.tensor([0.0, 0.0, 0.4], dtype=torch.float64), x) - 0.1) < 1e-12
    assert oracle.rel_err(torch.zeros(3), torch.zeros(3)) == 0.0
