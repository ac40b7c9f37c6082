"""GPU parity of raf.op.l2norm, raf.op.fuse_tensor and raf.op.defuse_tensor, called through the
C ABI.  l2norm: within one unit in the last place of the output dtype of the float64 oracle (the
kernel accumulates in float64 and rounds once; a tie in the last place may fall either way) and
bit-identical from run to run.  fuse / defuse: byte-exact."""
import numpy as np
import pytest
import torch

from oracle import halfs, tensor_ops
from tests.helpers import rng_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

NORM_SIZES = [0, 1, 2, 3, 4, 5, 7, 8, 9, 255, 256, 257, 4099, 16383, 16384, 16385, 65537, 1_000_003, 5_000_000]
ULP = {torch.float32: 2.0 ** -23, torch.float64: 2.0 ** -52, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def _norm_input(n, dtype, seed):
    x = rng_for(100, seed, 0).standard_normal(n) * 0.02
    if dtype == torch.bfloat16:
        bits = halfs.f32_to_bf16_bits(x.astype(np.float32))
        return bits, torch.from_numpy(bits.view(np.int16).copy()).to(DEV).view(torch.bfloat16)
    npdt = {torch.float32: np.float32, torch.float64: np.float64, torch.float16: np.float16}[dtype]
    a = x.astype(npdt)
    return a, torch.from_numpy(a).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
def test_l2norm_against_oracle(native_libs, dtype):
    from raf_amd import kernels

    for k, n in enumerate(NORM_SIZES):
        a, t = _norm_input(n, dtype, k)
        out = kernels.l2norm(t)
        assert out.dtype == dtype and out.dim() == 0
        got = float(out.double().cpu())
        want = tensor_ops.l2norm_f64(a)
        assert abs(got - want) <= ULP[dtype] * want, (n, got, want)
        again = kernels.l2norm(t)
        assert torch.equal(out, again) or n == 0 or bool(torch.isnan(out))  # run-to-run identical


def test_l2norm_special_values_and_views(native_libs):
    from raf_amd import kernels

    assert float(kernels.l2norm(torch.tensor([3.0, 4.0], device=DEV))) == 5.0
    assert float(kernels.l2norm(torch.tensor([3e30, 4e30], device=DEV))) == pytest.approx(5e30, rel=2e-7)
    assert float(kernels.l2norm(torch.tensor([60000.0, 60000.0], device=DEV, dtype=torch.float16))) == float("inf")
    assert np.isnan(float(kernels.l2norm(torch.tensor([1.0, float("nan")], device=DEV))))
    assert float(kernels.l2norm(torch.full((1 << 20,), 0.5, device=DEV))) == 512.0
    assert float(kernels.l2norm(torch.zeros(0, device=DEV))) == 0.0
    # a view that is only 4-byte aligned takes the element-wise path: same value
    base = torch.randn(100_001, device=DEV)
    a, b = kernels.l2norm(base[1:]), kernels.l2norm(base[1:].clone())
    assert torch.equal(a, b)
    # multi-dimensional input (the reference's test shape, test_tvm_reduce.py:199)
    x = torch.randn(2, 3, 4, device=DEV)
    assert float(kernels.l2norm(x)) == pytest.approx(float(torch.sqrt(torch.sum(x * x))), rel=1e-6)


def test_l2norm_beyond_two_to_the_31_elements(native_libs):
    """64-bit element counts: 2^31 + 12345 halves and quarters, whose sum of squares is exact."""
    import math
    from raf_amd import kernels

    n = 2 ** 31 + 12345
    x = torch.full((n,), 0.5, device=DEV, dtype=torch.float16)
    x[-7:] = 0.25
    want = math.sqrt((n - 7) * 0.25 + 7 * 0.0625)
    got = kernels.l2norm(x)
    assert float(got) == float(np.float16(want))
    del x, got
    y = torch.full((n,), 0.5, device=DEV)
    y[-7:] = 0.25
    assert float(kernels.l2norm(y)) == float(np.float32(want))


def test_l2norm_argument_errors(native_libs):
    from raf_amd import kernels

    with pytest.raises(TypeError):
        kernels.l2norm(torch.zeros(4, device=DEV, dtype=torch.int32))
    with pytest.raises(ValueError):
        kernels.l2norm(torch.zeros(4))
    x = torch.zeros(100_000, device=DEV)
    with pytest.raises(native_libs.RafHipError, match="workspace"):
        kernels.l2norm(x, workspace=torch.empty(8, dtype=torch.uint8, device=DEV))
    lib = native_libs.optim()
    assert lib.rafhip_l2norm(x.data_ptr(), 7, 4, x.data_ptr(), None, 0, None) == native_libs.RAFHIP_ERR_UNSUPPORTED
    assert lib.rafhip_l2norm_workspace_bytes(16384) == 0 and lib.rafhip_l2norm_workspace_bytes(16385) == 256


# ------------------------------------------------------------------------------- fuse / defuse
SHAPE_LISTS = {
    "mixed": [(3, 5), (7,), (0,), (2, 2, 2), (), (1025,), (65536,), (65537,), (300, 301)],
    "one": [(12345,)],
    "many small": [(int(n),) for n in np.random.default_rng(5).integers(1, 300, 500)],
}


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.uint8, np.float64])
@pytest.mark.parametrize("case", list(SHAPE_LISTS))
def test_fuse_and_defuse_are_byte_exact(native_libs, dtype, case):
    from raf_amd import kernels

    rng = np.random.default_rng(21)
    shapes = SHAPE_LISTS[case]
    data = [rng.integers(0, 256, int(np.prod(s, dtype=np.int64)) * np.dtype(dtype).itemsize, dtype=np.uint8)
            .view(dtype).reshape(s) for s in shapes]
    want = tensor_ops.fuse_tensor(data)
    parts = [torch.from_numpy(a.reshape(-1).view(np.uint8).copy()).to(DEV) for a in data]
    plan = kernels.FusePlan([p.numel() for p in parts], DEV)
    assert plan.total_bytes == want.nbytes
    flat = torch.full((plan.total_bytes + 64,), 0xAB, dtype=torch.uint8, device=DEV)
    plan.fuse(parts, flat[:plan.total_bytes])
    got = flat.cpu().numpy()
    assert np.array_equal(got[:want.nbytes], want.view(np.uint8))
    assert (got[want.nbytes:] == 0xAB).all(), "wrote past the end of the flat buffer"
    # and back, into fresh tensors surrounded by guard bytes
    backing = [torch.full((p.numel() + 32,), 0xCD, dtype=torch.uint8, device=DEV) for p in parts]
    outs = [b[16:16 + p.numel()] for b, p in zip(backing, parts)]
    plan.defuse(flat[:plan.total_bytes], outs)
    sizes, shp, idx = tensor_ops.defuse_args(data)
    back = tensor_ops.defuse_tensor(want, sizes, shp, idx)
    for b, o, a in zip(backing, outs, back):
        h = b.cpu().numpy()
        assert np.array_equal(h[16:16 + o.numel()], np.ascontiguousarray(a).reshape(-1).view(np.uint8))
        assert (h[:16] == 0xCD).all() and (h[16 + o.numel():] == 0xCD).all()
    plan.close()


def test_fuse_every_relative_alignment(native_libs):
    """Source and destination offsets in every combination modulo 16, lengths around the vector
    width: head, body and tail paths of the copy."""
    from raf_amd import kernels

    rng = np.random.default_rng(22)
    for n in (1, 15, 16, 17, 31, 100, 4096 + 5):
        plan = kernels.FusePlan([n], DEV)
        src_backing = torch.from_numpy(rng.integers(0, 256, n + 64, dtype=np.uint8)).to(DEV)
        for so in range(16):
            for do in (0, 1, 3, 4, 8, 13):
                dst_backing = torch.zeros(n + 64, dtype=torch.uint8, device=DEV)
                plan.fuse([src_backing[so:so + n]], dst_backing[do:do + n])
                assert torch.equal(dst_backing[do:do + n], src_backing[so:so + n]), (n, so, do)
                assert int(dst_backing[:do].sum()) == 0 and int(dst_backing[do + n:].sum()) == 0
        plan.close()


def test_fuse_large_list_and_pointer_changes(native_libs):
    """A BERT-base-sized fp32 list (streaming path), the same plan reused with other tensors."""
    from raf_amd import kernels, shapes

    sizes = shapes.numels(shapes.bert_base_shapes())
    plan = kernels.FusePlan([4 * n for n in sizes], DEV)
    for seed in (1, 2):
        gen = torch.Generator(DEV).manual_seed(seed)
        parts = [torch.randn(n, device=DEV, generator=gen) for n in sizes]
        flat = torch.empty(sum(sizes), device=DEV)
        plan.fuse(parts, flat)
        assert torch.equal(flat, torch.cat(parts))
        outs = [torch.empty_like(p) for p in parts]
        plan.defuse(flat, outs)
        assert all(torch.equal(a, b) for a, b in zip(parts, outs))
    plan.close()


def test_fuse_empty_and_errors(native_libs):
    from raf_amd import kernels

    empty = kernels.FusePlan([], DEV)
    assert empty.total_bytes == 0
    empty.fuse([], torch.empty(0, dtype=torch.uint8, device=DEV))
    zeros = kernels.FusePlan([0, 0], DEV)
    z = torch.empty(0, dtype=torch.uint8, device=DEV)
    zeros.fuse([z, z], z)
    plan = kernels.FusePlan([8, 4], DEV)
    a, b = torch.zeros(8, dtype=torch.uint8, device=DEV), torch.zeros(4, dtype=torch.uint8, device=DEV)
    with pytest.raises(ValueError):
        plan.fuse([a], torch.zeros(12, dtype=torch.uint8, device=DEV))
    with pytest.raises(ValueError):
        plan.fuse([a, b], torch.zeros(11, dtype=torch.uint8, device=DEV))
    with pytest.raises(ValueError):
        plan.fuse([b, a], torch.zeros(12, dtype=torch.uint8, device=DEV))
    import ctypes
    lib = native_libs.optim()
    h = ctypes.c_void_p(None)
    neg = (ctypes.c_int64 * 1)(-1)
    assert lib.rafhip_fuse_plan_create(1, neg, ctypes.byref(h)) == native_libs.RAFHIP_ERR_INVALID_ARG


# ------------------------------------------------------------------- through dialect dispatch
def test_ops_through_dialect_dispatch(native_libs):
    """raf_amd.op.l2norm / fuse_tensor / defuse_tensor: declare -> dispatch to the hip dialect ->
    OpEnv -> Execute, with outputs allocated from what declare produced."""
    from raf_amd import op

    x = torch.randn(2, 3, 4, device=DEV)
    out = op.l2norm(x)
    assert out.shape == () and out.dtype == torch.float32
    assert float(out) == pytest.approx(float(tensor_ops.l2norm_f64(x.cpu().numpy())), rel=2e-7)
    big = torch.randn(300_001, device=DEV, dtype=torch.float64)
    assert float(op.l2norm(big)) == pytest.approx(tensor_ops.l2norm_f64(big.cpu().numpy()), rel=1e-14)

    data = [torch.randn(s, device=DEV) for s in [(3, 5), (7,), (0,), (2, 2, 2), (), (70001,)]]
    flat = op.fuse_tensor(data)
    host = [t.cpu().numpy() for t in data]
    assert flat.shape == (sum(t.numel() for t in data),)
    assert np.array_equal(flat.cpu().numpy(), tensor_ops.fuse_tensor(host))
    sizes, shapes, idx = tensor_ops.defuse_args(host)
    back = op.defuse_tensor(flat, sizes, shapes, idx)
    assert len(back) == len(data)
    for a, b in zip(data, back):
        assert a.shape == b.shape and torch.equal(a, b)
    # half-precision lists keep their dtype
    h = [torch.randn(5, device=DEV).half(), torch.randn(3, device=DEV).half()]
    fh = op.fuse_tensor(h)
    assert fh.dtype == torch.float16 and torch.equal(fh, torch.cat(h))
    with op.with_dialect("cuda"):  # no such dialect here: nothing to dispatch to
        with pytest.raises(native_libs.RafError, match="Cannot find a valid dispatch"):
            op.l2norm(torch.randn(9, device=DEV))


def test_l2norm_golden_fixture(native_libs):
    """Stored l2norm results (four dtypes): equal, or one unit in the last place apart where the
    float64 sums differ in their last bits."""
    from raf_amd import kernels
    from tests.golden import make_fixtures as mf

    z = np.load(mf.HERE / "mixed_kat.npz")
    tdt = {"float32": torch.float32, "float64": torch.float64, "float16": torch.float16, "bfloat16": torch.bfloat16}
    idt = {"float32": np.int32, "float64": np.int64, "float16": np.int16, "bfloat16": np.int16}
    for dt in mf.NORM_DTYPES:
        for k, n in enumerate(mf.NORM_SIZES):
            a = mf.norm_input(n, dt, k)
            t = (torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16) if dt == "bfloat16"
                 else torch.from_numpy(a).to(DEV))
            got = kernels.l2norm(t).cpu().view(-1).view({2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])
            want = np.frombuffer(z[f"l2norm/{dt}/{n}"].tobytes(), dtype=idt[dt])
            assert abs(int(got[0]) - int(want[0])) <= 1, (dt, n)


@pytest.mark.parametrize("shape", [(64, 128), (128, 256)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_tensor_fusion_and_defusion(native_libs, shape, dtype):
    """The reference's own test of the two ops (tests/python/op/cuda/test_cuda_memory.py:13-43):
    the same tensor fused with itself and defused again, here with random data and exact equality."""
    from raf_amd import op

    size = shape[0] * shape[1]
    sizes = [size, size]
    tuple_shape = shape + shape
    shape_indices = [len(shape), 2 * len(shape)]
    x = torch.randn(shape, device=DEV).to(dtype)
    with op.with_dialect(["tvm", "hip"]):
        x_2 = op.fuse_tensor([x, x])
        x_3 = op.defuse_tensor(x_2, sizes, tuple_shape, shape_indices)
    assert x_2.shape == (2 * size,) and x_2.dtype == dtype
    assert len(x_3) == 2 and all(y.shape == x.shape and torch.equal(y, x) for y in x_3)


def test_fuse_and_defuse_on_a_requested_copy_stream(native_libs):
    """With the executor serving OpEnv::RequestStream, fuse_tensor / defuse_tensor run on the copy
    streams they request (the reference's tags, src/op/dialect/cuda/memory.cc:34, :89), ordered
    against the current stream on both sides: producers enqueued before the op and consumers
    enqueued after it, all on the current stream, see the right bytes."""
    from raf_amd import op

    parts = [torch.zeros(n, device=DEV) for n in (1 << 20, 70_001, 3, 1 << 22)]
    host = None
    op.serve_stream_requests(True)
    try:
        for rep in range(3):
            for k, t in enumerate(parts):  # producers on the current stream, right before the op
                t.fill_(float(10 * rep + k))
            flat = op.fuse_tensor(parts)
            total = flat.double().sum()  # a consumer on the current stream, right after the op
            want = sum(float(10 * rep + k) * t.numel() for k, t in enumerate(parts))
            assert float(total) == want
            flat.mul_(2.0)
            sizes, shapes, idx = tensor_ops.defuse_args([t.cpu().numpy() for t in parts])
            back = op.defuse_tensor(flat, sizes, shapes, idx)
            for k, b in enumerate(back):
                assert torch.equal(b, parts[k] * 2.0)
    finally:
        op.serve_stream_requests(False)
    # and without it the same results on the current stream
    flat = op.fuse_tensor(parts)
    assert torch.equal(flat, torch.cat([t.reshape(-1) for t in parts]))
