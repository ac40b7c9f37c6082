"""The benchmark configurations at their full sizes, and the operator front end, on the GPU.

Configurations 2-4 are compared element by element with the C restatement of the oracle (itself
pinned to the NumPy oracle).  Configuration 5 (GPT-2 1.5B, 100 steps, 25 GB resident) is too large
for a CPU oracle inside a test: whole tensors picked from its list are followed through all 100
steps against the oracle (tensors are independent, so they see exactly the full-size run), and
every other tensor is covered by size-independent properties."""
import numpy as np
import pytest
import torch

from oracle.lans_f64 import LansHParams
from tests.helpers import max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _gen(sizes, seed, g16=False, zero_state=True, loss_scale=1024.0):
    """Seeded synthetic tensors generated on the GPU: w~N(0,.02), g~N(0,1e-3) (fp16: times the loss
    scale), m~N(0,1e-4), v=|N(0,1e-6)| or zero state."""
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed)
    g, w, m, v = [], [], [], []
    for n in sizes:
        gt = torch.randn(n, device=DEV, generator=gen) * 1e-3
        g.append((gt * loss_scale).half() if g16 else gt)
        w.append(torch.randn(n, device=DEV, generator=gen) * 0.02)
        if zero_state:
            m.append(torch.zeros(n, device=DEV))
            v.append(torch.zeros(n, device=DEV))
        else:
            m.append(torch.randn(n, device=DEV, generator=gen) * 1e-4)
            v.append((torch.randn(n, device=DEV, generator=gen) * 1e-6).abs())
    return g, w, m, v


def _host(ts):
    return [t.cpu().numpy() for t in ts]


def _run_config(sizes, seed, hp, step, c_oracle, g16=False, zero_state=True, threads=16):
    from raf_amd import kernels

    g, w, m, v = _gen(sizes, seed, g16, zero_state)
    hg, hw, hm, hv = _host(g), _host(w), _host(m), _host(v)
    plan = kernels.LansPlan(sizes, g[0].dtype, DEV)
    khp = kernels.make_hparams(hp.learning_rate, hp.beta1, hp.beta2, hp.eps, hp.bias_correction,
                               hp.weight_decay, hp.grad_averaging, hp.mode, hp.normalize_grad,
                               hp.grad_unscale)
    plan.step(g, w, m, v, torch.tensor(float(step), device=DEV), khp)
    torch.cuda.synchronize()
    norms = plan.read_norms()
    onorms = c_oracle.lans_step_inplace(hg, hw, hm, hv, step, hp, threads=threads)
    worst = {"w": 0.0, "m": 0.0, "v": 0.0}
    mismatched = 0
    for t in range(len(sizes)):
        for q, dev_t, ref in (("w", w[t], hw[t]), ("m", m[t], hm[t]), ("v", v[t], hv[t])):
            got = dev_t.cpu().numpy()
            worst[q] = max(worst[q], max_rel_err(got, ref))
            mismatched += int((got != ref).sum())
    print(f"max rel err {worst}, elements not bit-equal to the oracle: {mismatched} of {3 * sum(sizes)}")
    assert max(worst.values()) <= 1e-5
    assert np.max(np.abs(norms - onorms) / np.where(onorms == 0, 1, onorms)) < 1e-10
    # step-1 property with zero state: ||w0 - w1|| == lr * ||w0|| per tensor
    return plan, (g, w, m, v), norms


def test_config2_bert_base_fp32(native_libs, c_oracle):
    from raf_amd import shapes

    sizes = shapes.numels(shapes.bert_base_shapes())
    _run_config(sizes, 2, LansHParams(), 1, c_oracle)


def test_config3_bert_large_fp16_grads(native_libs, c_oracle):
    from raf_amd import shapes

    sizes = shapes.numels(shapes.bert_large_shapes())
    _run_config(sizes, 3, LansHParams(grad_unscale=1.0 / 1024), 1, c_oracle, g16=True)


def test_config4_two_thousand_small_tensors(native_libs, c_oracle):
    from raf_amd import shapes

    sizes = shapes.log_uniform_numels()
    _run_config(sizes, 4, LansHParams(), 2, c_oracle, zero_state=False)


def test_config5_gpt2_hundred_steps_full_size(native_libs, c_oracle):
    from raf_amd import kernels, shapes

    sizes = shapes.numels(shapes.gpt2_shapes())
    assert sum(sizes) == 1_557_611_200
    hp = LansHParams()
    g, w, m, v = _gen(sizes, 5)
    # tensors followed on the CPU: position embedding, first block's ln_1.weight, c_attn.bias,
    # attn.c_proj.weight, last block's c_fc.bias, final LayerNorm bias
    picks = [1, 2, 5, 6, 2 + 47 * 12 + 9, 579]
    ref = {t: ([g[t].cpu().numpy()], [w[t].cpu().numpy()], [m[t].cpu().numpy()], [v[t].cpu().numpy()])
           for t in picks}
    w0_norm = torch.stack([x.double().norm() for x in w]).cpu().numpy()
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    khp = kernels.make_hparams()
    step_t = torch.zeros((), device=DEV)
    first = None
    for s in range(1, 101):
        step_t.fill_(float(s))
        plan.step(g, w, m, v, step_t, khp)
        if s == 1:
            torch.cuda.synchronize()
            first = plan.read_norms()
    torch.cuda.synchronize()
    last = plan.read_norms()
    # properties over all 580 tensors
    assert np.allclose(first[:, 1], w0_norm, rtol=1e-10)          # ||w|| the kernels saw at step 1
    assert np.allclose(first[:, 2], first[:, 3], rtol=1e-9)       # step 1: u_m == u_g
    for arrs in (w, m, v):  # all 580 tensors: a norm is finite only if every element is
        assert bool(torch.isfinite(torch.stack(torch._foreach_norm(arrs))).all())
    assert np.isfinite(last).all() and (last > 0).all()
    # picked tensors: all 100 steps against the oracle
    for t in picks:
        hg, hw, hm, hv = ref[t]
        for s in range(1, 101):
            n = c_oracle.lans_step_inplace(hg, hw, hm, hv, s, hp, threads=8)
        assert max_rel_err(w[t].cpu().numpy(), hw[0]) <= 1e-4, t
        assert max_rel_err(m[t].cpu().numpy(), hm[0]) <= 1e-4, t
        assert max_rel_err(v[t].cpu().numpy(), hv[0]) <= 1e-4, t
        assert np.max(np.abs(last[t] - n[0]) / n[0]) < 1e-9, t


# ------------------------------------------------------------------ operator front end
def test_op_sgd_through_dialect_dispatch(native_libs):
    from oracle import sgd_f32
    from raf_amd import op

    r = np.random.default_rng(8)
    x0, dx, v0 = (r.normal(0, s, (33, 65)).astype(np.float32) for s in (.02, 1e-3, 1e-3))
    tx, tdx, tv = (torch.from_numpy(a).to(DEV) for a in (x0, dx, v0))
    v1, x1 = op.sgd(tx, tdx, tv, 0.01, 0.9)  # (v1, x1) order of the reference op
    ov, ox = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    assert np.array_equal(v1.cpu().numpy(), ov) and np.array_equal(x1.cpu().numpy(), ox)
    assert np.array_equal(tx.cpu().numpy(), x0)
    with op.with_dialect("tvm"):  # pinning a dialect that is not there leaves nothing to dispatch to
        from raf_amd import _lib

        op.clear_op_env_cache()
        with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch"):
            op.sgd(tx, tdx, tv, 0.01, 0.9)


def test_optim_classes_follow_reference_semantics(native_libs):
    from oracle import lans_f64, sgd_f32
    from raf_amd import optim

    r = np.random.default_rng(9)
    shapes_ = [(6, 3, 5, 5), (6,), (10, 1536), (10,)]  # the small CNN of the reference's tests
    ws = [r.normal(0, .1, s).astype(np.float32) for s in shapes_]
    # SGD: lr .1, momentum .01, 10 iterations (tests/python/optim/test_sgd.py:80-125)
    # both the per-parameter op loop of the reference and the one-launch multi-tensor path
    params = [torch.from_numpy(a.copy()).to(DEV) for a in ws]
    params_mt = [torch.from_numpy(a.copy()).to(DEV) for a in ws]
    sgd = optim.SGD(params, 0.1, 0.01, multi_tensor=False)
    sgd_mt = optim.SGD(params_mt, 0.1, 0.01)
    hx = [a.copy() for a in ws]
    hv = [np.zeros_like(a) for a in ws]
    for _ in range(10):
        grads = [r.normal(0, 1, s).astype(np.float32) for s in shapes_]
        for p, q, gr in zip(params, params_mt, grads):
            p.grad = torch.from_numpy(gr).to(DEV)
            q.grad = torch.from_numpy(gr).to(DEV)
        sgd.step()
        sgd_mt.step()
        for i, gr in enumerate(grads):
            hv[i], hx[i] = sgd_f32.sgd_step(hx[i], gr, hv[i], 0.1, 0.01)
    for p, q, a in zip(params, params_mt, hx):
        assert np.array_equal(p.cpu().numpy(), a) and np.array_equal(q.cpu().numpy(), a)
    # a half-precision model: fp32 master weights and velocities, parameters are their narrowing
    from oracle import halfs
    half = [torch.from_numpy(a.copy()).to(DEV).to(torch.bfloat16) for a in ws]
    sgd_h = optim.SGD(half, 0.1, 0.01)
    mx = [p.float().cpu().numpy() for p in half]
    mv = [np.zeros_like(a) for a in mx]
    for _ in range(3):
        gb = [halfs.f32_to_bf16_bits(r.normal(0, 1, s).astype(np.float32)) for s in shapes_]
        for p, g in zip(half, gb):
            p.grad = torch.from_numpy(g.view(np.int16)).to(DEV).view(torch.bfloat16)
        sgd_h.step()
        mx, mv, mp = sgd_f32.sgd_list_step(mx, gb, mv, 0.1, 0.01, "bfloat16")
    for (p, w, v), a, b, c in zip(sgd_h.params, mx, mv, mp):
        assert np.array_equal(w.cpu().numpy(), a) and np.array_equal(v.cpu().numpy(), b)
        assert np.array_equal(p.view(torch.int16).cpu().numpy().view(np.uint16), c.reshape(p.shape))
    # LANS: defaults, step counter starts at 1 and advances per call (lans.py:66, :103)
    params = [torch.from_numpy(a.copy()).to(DEV) for a in ws]
    lans = optim.LANS(params)
    hw = [a.copy() for a in ws]
    hm = [np.zeros_like(a) for a in ws]
    hvv = [np.zeros_like(a) for a in ws]
    for it in range(4):
        grads = [r.normal(0, 1e-2, s).astype(np.float32) for s in shapes_]
        for p, gr in zip(params, grads):
            p.grad = torch.from_numpy(gr).to(DEV)
        lans.step()
        hw, hm, hvv, _ = lans_f64.lans_step(grads, hw, hm, hvv, it + 1, lans_f64.LansHParams())
    assert lans._step == 5
    for p, a in zip(params, hw):
        assert p.shape == a.shape and max_rel_err(p.cpu().numpy(), a) <= 1e-5
    for (_, _, m, v), a, b in zip(lans.params, hm, hvv):
        assert max_rel_err(m.cpu().numpy(), a) <= 1e-5 and max_rel_err(v.cpu().numpy(), b) <= 1e-5


def test_op_lans_fp16_gradients_with_unscale(native_libs):
    from oracle import lans_f64
    from raf_amd import op
    from tests.helpers import lans_inputs

    sizes = [100, 4097]
    g, w, m, v = lans_inputs(sizes, cfg=90, g16=True)
    tl = [torch.from_numpy(a).to(DEV) for a in g + w + m + v]
    op.set_lans_grad_unscale(1.0 / 1024)
    try:
        out = op.lans(tl, torch.tensor(3.0, device=DEV), 1e-3, 0.9, 0.999, 1e-6, True, 0.01, True, True, True)
    finally:
        op.set_lans_grad_unscale(1.0)
    assert out[2] is tl[2]  # the output list is the input list: in-place op
    ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, 3, lans_f64.LansHParams(grad_unscale=1.0 / 1024))
    for t in range(2):
        assert max_rel_err(tl[2 + t].cpu().numpy(), ow[t]) <= 1e-5
        assert max_rel_err(tl[4 + t].cpu().numpy(), om[t]) <= 1e-5
        assert max_rel_err(tl[6 + t].cpu().numpy(), ov[t]) <= 1e-5
        assert np.array_equal(tl[t].cpu().numpy(), g[t])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_op_lans_mixed_and_half_precision_optimizer(native_libs, dtype):
    """The extension op through dialect dispatch, and raf_amd.optim.LANS on a half-precision model:
    fp32 master weights follow the oracle, the model's parameters are their 16-bit narrowing."""
    from oracle import halfs, lans_f64
    from raf_amd import op, optim
    from tests.helpers import lans_inputs

    name = "float16" if dtype == torch.float16 else "bfloat16"
    sizes = [100, 4097, 20000]
    _, w, m, v = lans_inputs(sizes, cfg=91)
    params = [torch.from_numpy(a).to(DEV).to(dtype).requires_grad_() for a in w]
    masters = [p.detach().float().cpu().numpy() for p in params]  # what the optimizer starts from
    grads = [(torch.randn(n, device=DEV, generator=torch.Generator(DEV).manual_seed(7 + i)) * 1e-3).to(dtype)
             for i, n in enumerate(sizes)]
    opt = optim.LANS(params)
    assert opt.mixed
    g_np = [(halfs.f32_to_bf16_bits(g.float().cpu().numpy()) if name == "bfloat16" else g.cpu().numpy())
            for g in grads]
    ow, om, ov = masters, [np.zeros_like(a) for a in masters], [np.zeros_like(a) for a in masters]
    for step in (1, 2, 3):
        for p, g in zip(params, grads):
            p.grad = g
        opt.step()
        ow, om, ov, op16, _ = lans_f64.lans_mixed_step(g_np, ow, om, ov, step, lans_f64.LansHParams(), name)
    for (p, wm, mm, vm), a, b, c in zip(opt.params, ow, om, ov):
        assert max_rel_err(wm.cpu().numpy(), a) <= 1e-5
        assert max_rel_err(mm.cpu().numpy(), b) <= 1e-5 and max_rel_err(vm.cpu().numpy(), c) <= 1e-5
        bits = p.detach().view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(bits, halfs.narrow_weight(wm.cpu().numpy(), name).view(np.uint16))
    # the op itself: picked by dispatch, output list is the input list
    tl = grads + [t[1] for t in opt.params] + [t[2] for t in opt.params] + [t[3] for t in opt.params] + \
        [p.data for p in params]
    out = op.lans_mixed(tl, torch.tensor(4.0, device=DEV), 1e-3, 0.9, 0.999, 1e-6, True, 0.01, True, True, True)
    assert out[7] is tl[7] and len(out) == 15
    with pytest.raises(native_libs.RafError, match="float16 or bfloat16"):
        op.lans_mixed(tl[:12] + [t.float() for t in tl[12:]], torch.tensor(4.0, device=DEV), 1e-3, 0.9, 0.999,
                      1e-6, True, 0.01, True, True, True)


@pytest.mark.parametrize("schedule", ["pipelined", "phased"])
def test_tensor_beyond_two_to_the_31_elements(native_libs, schedule):
    """Element counts are 64-bit end to end (the reference's are int: lans.cc:57).  One tensor of
    2049 * 2^20 = 2,148,532,224 elements built as 2049 copies of a 2^20-element block, followed by
    a small tensor.  Without gradient normalisation the trust ratios ||w|| / ||u|| of the tiled
    tensor equal the block's, so every copy must carry the block's result: copies bitwise equal to
    one another (every chunk indexed correctly), the first one within tolerance of the oracle on
    the block, and the norms sqrt(2049) times the block's."""
    from oracle import lans_f64
    from raf_amd import kernels
    from tests.helpers import lans_inputs

    P, K = 1 << 20, 2049
    hp = lans_f64.LansHParams(normalize_grad=False, grad_unscale=1 / 1024)
    g, w, m, v = lans_inputs([P, 1000], cfg=400, g16=True)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    big = lambda a: dev(a).repeat(K)
    tg, tw, tm, tv = ([big(x[0]), dev(x[1])] for x in (g, w, m, v))
    assert tw[0].numel() == P * K > 2 ** 31
    plan = kernels.LansPlan([P * K, 1000], torch.float16, DEV)
    plan.set_schedule(schedule)
    plan.step(tg, tw, tm, tv, torch.tensor(3.0, device=DEV), kernels.make_hparams(normalize_grad=False,
                                                                                  grad_unscale=1 / 1024))
    torch.cuda.synchronize()
    norms = plan.read_norms()
    ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 3, hp)
    for got, want in ((tw, ow), (tm, om), (tv, ov)):
        tiles = got[0].view(K, P)
        assert torch.equal(tiles, tiles[0].expand(K, P)), "copies of the block differ"
        assert max_rel_err(tiles[0].cpu().numpy(), want[0]) <= 1e-5
        assert max_rel_err(got[1].cpu().numpy(), want[1]) <= 1e-5
    assert np.allclose(norms[0], on[0] * np.sqrt(K), rtol=1e-12, atol=0)
    assert np.allclose(norms[1], on[1], rtol=1e-12, atol=0)
    assert torch.equal(tg[0][-P:], dev(g[0])), "gradients must stay untouched"
    plan.close()
