"""GPU parity of dialect fusion: the operator sequence of the reference's traced SGD optimizer
(python/raf/optim/sgd.py:192-200), built as a graph, rewritten by the FuseDialect pass with the
`hip` dialect's `sgd_update` pattern and run as one primitive function through the C ABI, must
give bit for bit what the four element-wise operators give one after the other (the fp32 oracle:
four separately rounded operations), in place on w and v."""
import numpy as np
import pytest
import torch

from oracle import halfs, sgd_f32
from tests.helpers import rng_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(shape, cfg, grad):
    n = int(np.prod(shape))
    w = rng_for(cfg, 0, 1).normal(0, 0.02, n).astype(np.float32).reshape(shape)
    d = rng_for(cfg, 0, 0).normal(0, 1e-3, n).astype(np.float32).reshape(shape)
    v = rng_for(cfg, 0, 2).normal(0, 1e-3, n).astype(np.float32).reshape(shape)
    if grad == "float16":
        d = d.astype(np.float16)
    elif grad == "bfloat16":
        d = halfs.f32_to_bf16_bits(d)
    return w, d, v


def _dev(a):
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16)
    return torch.from_numpy(a.copy()).to(DEV)


@pytest.mark.parametrize("grad", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("shape", [(1,), (3,), (1025,), (1024, 1024), (30522, 7), (5, 3, 2, 7)])
def test_fused_traced_update_is_bit_exact(native_libs, grad, shape):
    from raf_amd import op

    w, d, v = _inputs(shape, 300, grad)
    tw, td, tv = _dev(w), _dev(d), _dev(v)
    w_ptr, v_ptr = tw.data_ptr(), tv.data_ptr()
    ow, ov = w.ravel(), v.ravel()
    for step in range(3):
        out, before, after = op.traced_sgd_update(tw, td, tv, 0.01, 0.9, return_ir=True)
        assert out is tw and tw.data_ptr() == w_ptr and tv.data_ptr() == v_ptr  # out=w, out=v
        (ow,), (ov,), _ = sgd_f32.sgd_list_step([ow], [d.ravel()], [ov], 0.01, 0.9)
    torch.cuda.synchronize()
    assert np.array_equal(tw.cpu().numpy().ravel().view(np.uint32), ow.view(np.uint32))
    assert np.array_equal(tv.cpu().numpy().ravel().view(np.uint32), ov.view(np.uint32))
    # what the pass did: four (five) base-op calls became one call of a primitive hip function
    assert "raf.op.subtract(" in before and "hip" not in before
    assert ("raf.op.cast(" in before) == (grad != "float32")
    for piece in ("Primitive=1", "Dialect=hip", "PatternName=sgd_update", "raf.op.hip.subtract(",
                  "raf.op.hip.add(", "raf.op.hip.multiply("):
        assert piece in after, piece
    assert "raf.op.subtract(" not in after and ("raf.op.hip.cast(" in after) == (grad != "float32")
    assert after.count("= fn (") == 1


def test_fused_update_equals_the_sgd_op(native_libs):
    """raf.op.sgd and the fused traced sequence are the same arithmetic (python/raf/_tvm_op/sgd.py:21-29
    against python/raf/optim/sgd.py:197-200)."""
    from raf_amd import op

    w, d, v = _inputs((4099,), 301, "float32")
    tw, td, tv = _dev(w), _dev(d), _dev(v)
    v1, x1 = op.sgd(tw, td, tv, 0.05, 0.8)
    upd = op.TracedSgdUpdate(tw, td, tv, 0.05, 0.8)
    assert upd.op == "raf.op.hip._fused_op"  # DispatchFusedOp's maker name (src/impl/op.cc:190-192)
    assert upd() is tw
    assert torch.equal(v1, tv) and torch.equal(x1, tw)
    v2, x2 = op.sgd(tw, td, tv, 0.05, 0.8)
    upd()  # bound once, run again on the same tensors
    assert torch.equal(v2, tv) and torch.equal(x2, tw)


def test_unfusable_graphs_find_no_backend(native_libs):
    from raf_amd import op
    from raf_amd._lib import RafError

    w = torch.zeros(16, dtype=torch.float64, device=DEV)
    with pytest.raises(RafError, match="Cannot find a valid dispatch for op raf.op.subtract"):
        op.traced_sgd_update(w, w.clone(), w.clone(), 0.1, 0.9)
    w32 = torch.zeros(16, device=DEV)
    with pytest.raises(RafError, match="differ in shape"):
        op.traced_sgd_update(w32, torch.zeros(1, device=DEV), w32.clone(), 0.1, 0.9)


def test_traced_update_trains_like_torch_sgd(native_libs):
    """The reference's test of its traced optimizer (tests/python/optim/test_sgd.py:151-172): a 2x2
    parameter under relu, random output gradients, 32 steps of with_sgd(0.1, 0.01) against
    torch.optim.SGD at 1e-4 -- here with the traced update taken through the fusion pass."""
    from raf_amd import op

    torch.manual_seed(0)
    shape = (2, 2)
    x_t = torch.nn.Parameter(torch.randn(*shape, device=DEV))
    t_opt = torch.optim.SGD([x_t], lr=0.1, momentum=0.01)
    x_m = x_t.detach().clone()
    v_m = torch.zeros_like(x_m)
    grad = torch.empty_like(x_m)
    update = op.TracedSgdUpdate(x_m, grad, v_m, 0.1, 0.01)
    for _ in range(32):
        dy = torch.randn(*shape, device=DEV)
        t_opt.zero_grad()
        torch.relu(x_t).backward(dy)
        t_opt.step()
        grad.copy_(dy * (x_m > 0))  # relu's gradient at our own parameter
        update()
        np.testing.assert_allclose(x_m.cpu().numpy(), x_t.detach().cpu().numpy(), rtol=1e-4, atol=1e-4)
