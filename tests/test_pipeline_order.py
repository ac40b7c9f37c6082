"""Host logic of the pipelined LANS schedule (no GPU): the work list must contain every unit of work
exactly once and respect the per-tensor order that makes the kernel's waits finite."""
import pytest

KIND_A, KIND_B, KIND_C, KIND_WHOLE, KIND_FIN_A, KIND_FIN_B = range(6)


STREAMED = 8  # flag added to the kind


def _normalise(order):
    """Strips the flag: returns the list of (base kind, tensor, chunk) and the set of tensors whose
    items are marked streamed."""
    out, streamed = [], set()
    for kind, t, c in order:
        base = kind & 7
        assert kind in (base, base | STREAMED)
        if kind & STREAMED:
            streamed.add(t)
            assert base in (KIND_A, KIND_B, KIND_C), "only data-moving items carry the streaming mark"
        out.append((base, t, c))
    return out, streamed


def _check(order, sizes, lib, stream_from=(256 << 20) // 12):
    # a tensor's chunk size (and first-pass unit) depends on its own element count
    n_chunks = [-(-n // lib.rafhip_lans_chunk_elements(n)) for n in sizes]
    n_units = [-(-n // lib.rafhip_lans_pass_a_unit_elements(n)) for n in sizes]
    order, streamed = _normalise(order)
    seen = {}
    for pos, (kind, t, c) in enumerate(order):
        assert 0 <= t < len(sizes) and sizes[t] > 0, "empty tensors contribute no work"
        assert (kind, t, c) not in seen, "duplicate work item"
        seen[(kind, t, c)] = pos
    for t in streamed:
        assert sizes[t] >= stream_from, "only tensors beyond the cache are streamed"
    for t, nc in enumerate(n_chunks):
        if nc == 0:
            continue
        if nc == 1:
            assert (KIND_WHOLE, t, 0) in seen
            assert not any((k, t, 0) in seen for k in (KIND_A, KIND_B, KIND_C, KIND_FIN_A, KIND_FIN_B))
            continue
        a = [seen[(KIND_A, t, u)] for u in range(n_units[t])]
        assert (KIND_A, t, n_units[t]) not in seen
        b = [seen[(KIND_B, t, c)] for c in range(nc)]
        cc = [seen[(KIND_C, t, c)] for c in range(nc)]
        fa, fb = seen[(KIND_FIN_A, t, 0)], seen[(KIND_FIN_B, t, 0)]
        assert max(a) < fa < min(b), f"tensor {t}: finish A must follow its chunks and precede pass B"
        assert max(b) < fb < min(cc), f"tensor {t}: finish B must follow its chunks and precede pass C"
    expect = sum(1 if nc == 1 else 2 * nc + nu + 2 for nc, nu in zip(n_chunks, n_units) if nc)
    assert len(order) == expect


@pytest.mark.parametrize("group", [0, 1, 100_000, 10**12])
def test_order_invariants(native_libs, group):
    from raf_amd import kernels, shapes

    lib = native_libs.optim()
    chunk, unit_a = lib.rafhip_lans_chunk_elements(1), lib.rafhip_lans_pass_a_unit_elements(1)
    big = 1 << 19  # from here on tensors are cut into larger chunks
    assert unit_a % chunk == 0 and lib.rafhip_lans_chunk_elements(big) > lib.rafhip_lans_chunk_elements(big - 1) == chunk
    assert lib.rafhip_lans_pass_a_unit_elements(big) % lib.rafhip_lans_chunk_elements(big) == 0
    lists = [
        [1, 3, 0, chunk - 1, chunk, chunk + 1, 5 * chunk + 7, 0, 2 * chunk, 17, unit_a, unit_a + 1, 3 * unit_a - 1,
         big - 1, big, big + 1, 3 * big + 5],
        shapes.log_uniform_numels(300, seed=7),
        shapes.numels(shapes.bert_base_shapes()),
        [],
        [0, 0],
        [23_000_000, 5000, 70_000],            # a streamed tensor with hardly anything beside it
        [40_000_000],                          # ... and alone
        [1 << 20] * 30 + [30_000_000] + [1 << 20] * 30 + [25_000_000],  # two streamed tensors among cached groups
    ]
    for sizes in lists:
        _check(kernels.pipeline_order(sizes, group), sizes, lib)


def test_order_invariants_on_random_lists(native_libs, monkeypatch):
    """The same invariants over a few hundred random lists: every mix of empty, one-chunk, small-chunk,
    large-chunk and cache-exceeding tensors, with random cache-group sizes, streaming thresholds and
    hold lengths."""
    import numpy as np

    from raf_amd import kernels

    lib = native_libs.optim()
    rng = np.random.default_rng(31)
    for case in range(300):
        n = int(rng.integers(1, 25))
        kinds = rng.integers(0, 6, n)
        sizes = []
        for k in kinds:
            if k == 0:
                sizes.append(int(rng.integers(0, 3)))                    # empty or tiny
            elif k == 1:
                sizes.append(int(rng.integers(1, 4097)))                 # one chunk
            elif k == 2:
                sizes.append(int(rng.integers(4097, 1 << 19)))           # small chunks
            elif k == 3:
                sizes.append(int(rng.integers(1 << 19, 6_000_000)))      # large chunks
            elif k == 4:
                sizes.append(int(rng.integers(6_000_000, 22_000_000)))   # long, still cached
            else:
                sizes.append(int(rng.integers(22_400_000, 60_000_000)))  # streamed
        group = int(rng.choice([0, 1, 50_000, 3_000_000, 13_000_000, 10**12]))
        stream_from = int(rng.choice([(256 << 20) // 12, 30_000, 1_000_000, 10**12]))
        hold = int(rng.choice([0, 3, 3072, 10**6]))
        try:
            _check(kernels.pipeline_order(sizes, group, stream_from_elements=stream_from, stream_hold_items=hold),
                   sizes, lib, stream_from)
        except AssertionError as e:
            raise AssertionError(f"case {case}: sizes {sizes}, group {group}: {e}") from e


def test_groups_bound_the_reuse_distance(native_libs):
    """Between a tensor's pass-A chunks and its pass-C chunks lie at most a few groups' worth of
    other tensors' work, which is what keeps the tensor in the Infinity Cache."""
    from raf_amd import kernels

    chunk = native_libs.optim().rafhip_lans_chunk_elements(1)
    sizes = [8 * chunk] * 40  # 40 equal tensors, group = 2 tensors
    order, _ = _normalise(kernels.pipeline_order(sizes, 16 * chunk))
    first_a = {t: min(i for i, (k, tt, _) in enumerate(order) if k == KIND_A and tt == t) for t in range(40)}
    last_c = {t: max(i for i, (k, tt, _) in enumerate(order) if k == KIND_C and tt == t) for t in range(40)}
    per_group = 2 * (2 * 8 + 1 + 2)
    for t in range(40):
        assert last_c[t] - first_a[t] <= 3 * per_group
    # one giant group degenerates into pass-major order: all of A, then all of B, then all of C
    order, _ = _normalise(kernels.pipeline_order(sizes, 10**12))
    kinds = [k for k, _, _ in order]
    assert max(i for i, k in enumerate(kinds) if k in (KIND_A, KIND_FIN_A)) < min(
        i for i, k in enumerate(kinds) if k == KIND_B)


def test_bert_large_group_structure(native_libs):
    from raf_amd import kernels, shapes

    sizes = shapes.numels(shapes.bert_large_shapes())
    order = kernels.pipeline_order(sizes)
    lib = native_libs.optim()
    _check(order, sizes, lib)
    assert sum(1 for k, _, _ in order if k == KIND_WHOLE) == sum(
        1 for n in sizes if 0 < n <= lib.rafhip_lans_chunk_elements(n))
    # the word embedding (31 M elements: 375 MB of w, m, v) is streamed, and its items are spread
    # over the list instead of standing at its head
    emb = [i for i, (k, t, _) in enumerate(order) if t == 0]
    assert all(k & STREAMED for k, t, _ in order if t == 0 and (k & 7) in (KIND_A, KIND_B, KIND_C))
    assert not any(k & STREAMED for k, t, _ in order if t != 0)
    assert emb[-1] > 0.9 * len(order) and emb[len(emb) // 2] > 0.3 * len(order)


def test_streamed_items_keep_clear_of_their_finish_items(native_libs):
    """What follows a finish item of a streamed tensor waits for it: the next streamed item comes
    only after a few items per workgroup of other work."""
    from raf_amd import kernels, shapes

    order = kernels.pipeline_order(shapes.numels(shapes.bert_large_shapes()))
    pos = {(k & 7): i for i, (k, t, _) in enumerate(order) if t == 0 and (k & 7) in (KIND_FIN_A, KIND_FIN_B)}
    for fin in pos.values():
        nxt = next(i for i in range(fin + 1, len(order)) if order[i][1] == 0)
        assert nxt - fin > 2 * 768
