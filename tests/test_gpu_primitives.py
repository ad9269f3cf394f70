"""GPU parity: scan / sort primitives, hash grid and rulebooks against the CPU oracle.
Integer structures are compared bit-exactly: the HIP grid numbers sites by first appearance
exactly like the oracle, so raw ids can be compared, and the canonical (sorted-by-coordinate)
form is checked as well."""
import ctypes

import numpy as np
import pytest
import torch

from workloads import scenes

pytestmark = pytest.mark.gpu
I64 = ctypes.c_int64


@pytest.fixture(scope="module")
def S():
    from sparseconvnet import SCN
    from sparseconvnet._lib import ensure_init

    ensure_init(0)
    return SCN


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


@pytest.mark.parametrize("n", [0, 1, 63, 1023, 1025, 2048, 2049, 32768, 32769, 100003, 3000000, 8388608, 8400001])
def test_scan(S, n):
    from sparseconvnet._lib import lib, ptr, stream_ptr

    rng = np.random.default_rng(n)
    a = rng.integers(0, 5, n).astype(np.int32)
    d_in = dev(a) if n else torch.empty(0, dtype=torch.int32, device="cuda")
    d_out = torch.empty_like(d_in)
    tot = torch.full((1,), -7, dtype=torch.int32, device="cuda")
    lib.insc_scan_exclusive_i32(ptr(d_in), ptr(d_out), I64(n), ptr(tot), stream_ptr())
    exp = np.concatenate([[0], np.cumsum(a)[:-1]]) if n else np.zeros(0)
    assert (d_out.cpu().numpy() == exp).all()
    assert int(tot.item()) == int(a.sum())
    if n:  # in place, as the library's own callers use it (short inputs take one workgroup, longer ones two launches, beyond 8.4 M values three)
        lib.insc_scan_exclusive_i32(ptr(d_in), ptr(d_in), I64(n), None, stream_ptr())
        assert (d_in.cpu().numpy() == exp).all()


@pytest.mark.parametrize("n,bits", [(1, 64), (1000, 16), (2048, 64), (50001, 40), (700000, 64), (300000, 3)])
def test_sort_stable(S, n, bits):
    from sparseconvnet._lib import lib, ptr, stream_ptr

    rng = np.random.default_rng(n + bits)
    hi = (1 << bits) - 1 if bits < 63 else (1 << 63) - 1
    # few distinct values in part of the range so that stability matters
    k = rng.integers(0, min(hi, 50) + 1, n).astype(np.uint64) if bits <= 16 else \
        rng.integers(0, hi, n, dtype=np.int64).astype(np.uint64)
    if bits == 64:
        k |= (rng.integers(0, 2, n).astype(np.uint64) << np.uint64(63))
    v = np.arange(n, dtype=np.int32)
    dk = torch.from_numpy(k.view(np.int64)).cuda()
    dv = dev(v)
    lib.insc_sort_pairs_u64(ptr(dk), ptr(dv), I64(n), bits, stream_ptr())
    order = np.argsort(k, kind="stable")
    assert (dv.cpu().numpy() == v[order]).all()
    assert (dk.cpu().numpy().view(np.uint64) == k[order]).all()


def _insert(S, pts, capacity=None):
    m = S.Metadata_3()
    m._bind(torch.device("cuda", 0))
    sc = m.scale((4096,) * 3, create_capacity=capacity or max(len(pts), 1))
    sop = m.insert(sc, dev(pts, torch.int32)) if len(pts) else torch.empty(0, dtype=torch.int32)
    return m, sc, sop


@pytest.mark.parametrize("case", ["dups", "unique", "batched"])
def test_grid_insert_matches_oracle(S, orc, case):
    rng = np.random.default_rng(11)
    if case == "dups":
        pts = np.concatenate([rng.integers(0, 12, (20000, 3)), np.zeros((20000, 1), np.int64)], 1)
    elif case == "unique":
        pts = scenes.boxes_scene(seed=3, n=20000)
    else:
        pts = np.concatenate([rng.integers(100, 140, (30000, 3)), rng.integers(0, 5, (30000, 1))], 1)
    pts = pts.astype(np.int32)
    m, sc, sop = _insert(S, pts)
    o_sop, o_sc, o_cnt = orc.grid_build(pts)
    assert sc.n == len(o_sc)
    assert (sop.cpu().numpy() == o_sop).all()
    got = sc.coords_view().cpu().numpy()
    assert (got == o_sc).all()
    assert (orc.canonical_sites(got) == orc.canonical_sites(np.unique(pts, axis=0))).all()
    assert (m.getSpatialLocations((4096,) * 3).numpy() == o_sc).all()


def test_grid_query_append_and_grow(S, orc):
    rng = np.random.default_rng(12)
    a = rng.integers(0, 30, (5000, 3)).astype(np.int32)
    a = np.concatenate([a, np.zeros((len(a), 1), np.int32)], 1)
    m, sc, sop = _insert(S, a, capacity=1024)  # forces a rehash (capacity < sites)
    b = rng.integers(0, 40, (9000, 3)).astype(np.int32)
    b = np.concatenate([b, np.zeros((len(b), 1), np.int32)], 1)
    sop_b = m.insert(sc, dev(b))
    # append-only numbering == oracle numbering of the concatenated list
    o_sop, o_sc, _ = orc.grid_build(np.concatenate([a, b], 0))
    assert sc.n == len(o_sc)
    assert (sop.cpu().numpy() == o_sop[:len(a)]).all()
    assert (sop_b.cpu().numpy() == o_sop[len(a):]).all()
    assert (sc.coords_view().cpu().numpy() == o_sc).all()
    # queries: hits, misses, out-of-range coordinates
    q = rng.integers(-2, 45, (20000, 3)).astype(np.int32)
    q = np.concatenate([q, np.zeros((len(q), 1), np.int32)], 1)
    q[:5, 0] = [70000, -1, 65536, 3, 3]
    out = torch.empty(len(q), dtype=torch.int32, device="cuda")
    from sparseconvnet._lib import lib, ptr, stream_ptr

    lib.insc_grid_query(sc.grid, ptr(dev(q)), I64(len(q)), ptr(out), stream_ptr())
    assert (out.cpu().numpy() == orc.grid_query(o_sc, q)).all()


@pytest.mark.parametrize("case", ["hot_cells", "scene", "batched_wide"])
def test_large_insert_built_by_partitions(S, orc, case):
    """An insert of more than 16 384 rows into an empty grid sorts its rows by table partition and builds each
    partition in LDS; the large insert that follows, into the grid that then holds sites, claims its slots
    in the table itself.  Ids, per-row sites and the table (queries) against the oracle; rows with the skip
    mark get -1."""
    from sparseconvnet._lib import lib, ptr, stream_ptr

    rng = np.random.default_rng(21)
    if case == "hot_cells":  # 1 728 cells hit by 300 000 rows: a few partitions take nearly every row
        a = np.concatenate([rng.integers(0, 12, (300000, 3)), np.zeros((300000, 1), np.int64)], 1).astype(np.int32)
        b = np.concatenate([rng.integers(6, 40, (70000, 3)), np.zeros((70000, 1), np.int64)], 1).astype(np.int32)
    elif case == "scene":
        pts = scenes.boxes_scene(seed=5, n=230000).astype(np.int32)
        a, b = pts[:150000], np.concatenate([pts[100000:140000], pts[150000:]], 0)
    else:
        a = np.concatenate([rng.integers(0, 65536, (200000, 3)), rng.integers(0, 32768, (200000, 1))], 1).astype(np.int32)
        b = np.concatenate([a[rng.integers(0, len(a), 30000)], a[:40000] ^ 1], 0).astype(np.int32)
    skip = np.zeros(len(a), bool)
    skip[rng.integers(0, len(a), 50)] = True
    a_in = a.copy()
    a_in[skip, 0] = np.iinfo(np.int32).min
    m, sc, sop = _insert(S, a_in, capacity=262144)
    o_sop, o_sc, _ = orc.grid_build(np.concatenate([a[~skip], b], 0))
    n_a = int((~skip).sum())
    got = sop.cpu().numpy()
    assert (got[skip] == -1).all()
    assert (got[~skip] == o_sop[:n_a]).all()
    assert sc.n == int(o_sop[:n_a].max()) + 1
    sop_b = m.insert(sc, dev(b))  # the grid holds sites now
    assert sc.n == len(o_sc)
    assert (sop_b.cpu().numpy() == o_sop[n_a:]).all()
    assert (sc.coords_view().cpu().numpy() == o_sc).all()
    q = np.concatenate([a[::7], b[::5], (a[:20000] + np.array([1, 0, 0, 0], np.int32)) & 65535], 0).astype(np.int32)
    q[:, 3] &= 32767
    out = torch.empty(len(q), dtype=torch.int32, device="cuda")
    lib.insc_grid_query(sc.grid, ptr(dev(q)), I64(len(q)), ptr(out), stream_ptr())
    assert (out.cpu().numpy() == orc.grid_query(o_sc, q)).all()


@pytest.mark.parametrize("shape", ["cube", "plane", "column"])
def test_grid_at_half_load_with_crowded_groups(S, orc, shape):
    """Scenes that crowd the table's groups of eight slots, at the highest load the grid allows (0.5): a solid
    cube (every z-run fills its group), a flat plane (every key wants position z & 7 = 5 of its group) and
    columns along z; inserted in one call and in two, then looked up (hits and misses)."""
    from sparseconvnet._lib import lib, ptr, stream_ptr

    rng = np.random.default_rng(3)
    if shape == "cube":
        g = np.stack(np.meshgrid(np.arange(64), np.arange(64), np.arange(64), indexing="ij"), -1).reshape(-1, 3) + 100
    elif shape == "plane":
        g = np.stack(np.meshgrid(np.arange(512), np.arange(512), [5], indexing="ij"), -1).reshape(-1, 3)
    else:
        g = np.stack(np.meshgrid(np.arange(16), np.arange(16), np.arange(1024), indexing="ij"), -1).reshape(-1, 3)
    pts = np.concatenate([g, np.zeros((len(g), 1), np.int64)], 1).astype(np.int32)[rng.permutation(len(g))]
    assert len(pts) == 262144
    o_sop, o_sc, _ = orc.grid_build(pts)
    for cut in (len(pts), 200000):
        m, sc, sop = _insert(S, pts[:cut], capacity=262144)  # 2^19 slots
        got = sop.cpu().numpy()
        if cut < len(pts):
            got = np.concatenate([got, m.insert(sc, dev(pts[cut:])).cpu().numpy()])
        assert sc.n == len(o_sc)
        assert (got == o_sop).all()
        assert (sc.coords_view().cpu().numpy() == o_sc).all()
        q = np.concatenate([pts[::3], pts[:30000] + np.array([0, 0, 1100, 0], np.int32)], 0).astype(np.int32)
        out = torch.empty(len(q), dtype=torch.int32, device="cuda")
        lib.insc_grid_query(sc.grid, ptr(dev(q)), I64(len(q)), ptr(out), stream_ptr())
        assert (out.cpu().numpy() == orc.grid_query(o_sc, q)).all()


def test_grid_rejects_bad_coordinate(S):
    from sparseconvnet._lib import InscError

    pts = np.array([[1, 2, 3, 0], [70000, 1, 1, 0]], np.int32)
    with pytest.raises(InscError):
        _insert(S, pts)
    pts = np.array([[1, 2, 3, 0], [1, -1, 1, 0]], np.int32)
    with pytest.raises(InscError):
        _insert(S, pts)


@pytest.mark.parametrize("scene", ["cfg1", "random", "border"])
def test_ssc_rulebook_matches_oracle(S, orc, scene):
    if scene == "cfg1":
        pts = scenes.boxes_scene(seed=1, n=20000)
    elif scene == "random":
        rng = np.random.default_rng(5)
        pts = np.concatenate([rng.integers(0, 20, (6000, 3)), rng.integers(0, 2, (6000, 1))], 1).astype(np.int32)
    else:  # sites on the coordinate borders: -1 and 65536 neighbours must not alias
        rng = np.random.default_rng(6)
        pts = np.concatenate([rng.choice([0, 1, 65534, 65535], (500, 3)), np.zeros((500, 1), np.int64)], 1).astype(np.int32)
    m, sc, _ = _insert(S, pts)
    m.ssc_rulebook((4096,) * 3)
    o_sop, o_sc, _ = orc.grid_build(pts)
    o_nbr, o_counts, o_pairs = orc.ssc_rules(o_sc)
    assert (sc.nbr.t[:sc.n].cpu().numpy() == o_nbr).all()
    counts, pairs = S.ssc_rulebook_lists(m, (4096,) * 3)
    assert (counts.numpy() == o_counts).all()
    assert (pairs.numpy() == o_pairs).all()
    can = orc.canonical_rules(counts.numpy(), pairs.numpy(), o_sc, o_sc)
    assert (can == orc.canonical_rules(o_counts, o_pairs, o_sc, o_sc)).all()
    # the processing order is a permutation of the sites
    assert (np.sort(sc.order.t[:sc.n].cpu().numpy()) == np.arange(sc.n)).all()


def test_ssc_rulebook_incremental_patch(S, orc):
    """Appending sites and patching the map equals building it from scratch."""
    pts = scenes.boxes_scene(seed=9, n=12000)
    m, sc, _ = _insert(S, pts[:7000])
    m.ssc_rulebook((4096,) * 3)
    m.insert(sc, dev(pts[7000:]))
    m.ssc_rulebook((4096,) * 3)
    _, o_sc, _ = orc.grid_build(pts)
    o_nbr, _, _ = orc.ssc_rules(o_sc)
    assert sc.n == len(o_sc)
    assert (sc.nbr.t[:sc.n].cpu().numpy() == o_nbr).all()
    assert (np.sort(sc.order.t[:sc.n].cpu().numpy()) == np.arange(sc.n)).all()


def _spread3(v):
    out = np.zeros_like(v)
    for b in range(8):
        out |= ((v >> np.uint64(b)) & np.uint64(1)) << np.uint64(3 * b)
    return out


@pytest.mark.parametrize("n_old,n_new", [(7000, 1), (7000, 63), (7000, 700), (40000, 3300), (9000, 8192), (9000, 8193)])
def test_order_append_sorts_the_new_sites(S, n_old, n_new):
    """insc_order_append against numpy: the sites of the last insert in the order of (64^3 block, neighbour
    pattern), equal keys by id; the inverse; the same sites grouped by their position inside the parent
    cell, each group in that order.  One site, fewer than a wavefront, a frame's worth, the most the
    workgroup sorts, and one more (which keep their id order)."""
    from sparseconvnet._lib import lib, ptr, stream_ptr

    rng = np.random.default_rng(n_new)
    pts = scenes.boxes_scene(seed=13, n=n_old + n_new).astype(np.int32)
    pts[:, :3] += rng.integers(0, 3, 3).astype(np.int32) * 64  # several 64^3 blocks
    pts[:, 3] = rng.integers(0, 2, len(pts))  # two batch entries
    m, sc, _ = _insert(S, pts[:n_old], capacity=n_old + n_new)
    m.ssc_rulebook((4096,) * 3)
    m.insert(sc, dev(pts[n_old:]))
    assert sc.n == n_old + n_new
    nbr = sc.nbr.ensure(sc.capacity(), keep=sc.nbr_n)
    lib.insc_rulebook_ssc3(sc.grid, I64(n_old), I64(n_new), ptr(nbr), 1, stream_ptr())
    offset = dev(rng.integers(0, 8, sc.n).astype(np.int32))
    order, pos, bo, bop = (torch.full((sc.n,), -5, dtype=torch.int32, device="cuda") for _ in range(4))
    lib.insc_order_append(sc.grid, ptr(nbr), ptr(offset), ptr(order), ptr(pos), ptr(bo), ptr(bop), I64(n_new),
                          stream_ptr())
    c = sc.coords_view().cpu().numpy()[n_old:].astype(np.uint64)
    has = nbr[:sc.n].view(-1, 27)[n_old:].cpu().numpy() >= 0
    pattern = (has.astype(np.uint64) << np.arange(27, dtype=np.uint64)).sum(1)
    mort = _spread3((c[:, 0] >> np.uint64(6)) & np.uint64(15)) | (_spread3((c[:, 1] >> np.uint64(6)) & np.uint64(15)) << np.uint64(1)) \
        | (_spread3((c[:, 2] >> np.uint64(6)) & np.uint64(15)) << np.uint64(2))
    key = ((c[:, 3] & np.uint64(1)) << np.uint64(39)) | (mort << np.uint64(27)) | pattern
    exp = n_old + (np.argsort(key, kind="stable") if n_new <= 8192 else np.arange(n_new))
    got = order.cpu().numpy()
    assert (got[:n_old] == -5).all()  # older sites are not touched
    assert (got[n_old:] == exp).all()
    if n_new <= 8192:  # the device-wide radix sort of insc_order_build orders them the same way
        order2 = torch.full((sc.n,), -5, dtype=torch.int32, device="cuda")
        lib.insc_order_build(sc.grid, ptr(nbr), I64(n_old), I64(n_new), ptr(order2), stream_ptr())
        assert (order2.cpu().numpy() == got).all()
    assert (pos.cpu().numpy()[exp] == n_old + np.arange(n_new)).all()
    off = offset.cpu().numpy()
    exp_bo = exp[np.argsort(off[exp] & 7, kind="stable")] if n_new <= 8192 else exp
    assert (bo.cpu().numpy()[n_old:] == exp_bo).all()
    assert (bop.cpu().numpy()[exp_bo] == n_old + np.arange(n_new)).all()


def test_down2_rulebook_matches_oracle(S, orc):
    pts = scenes.boxes_scene(seed=2, n=20000)
    m, sc, _ = _insert(S, pts)
    fine, coarse, d = m.down_rulebook((4096,) * 3, (2048,) * 3)
    _, o_sc, _ = orc.grid_build(pts)
    parent, off, cc = orc.down2_rules(o_sc)
    assert coarse.n == len(cc)
    assert (d.parent.t[:fine.n].cpu().numpy() == parent).all()
    assert (d.offset.t[:fine.n].cpu().numpy() == off).all()
    assert (coarse.coords_view().cpu().numpy() == cc).all()
    child = d.child.t[:coarse.n].cpu().numpy()
    exp = np.full((len(cc), 8), -1, np.int32)
    exp[parent, off] = np.arange(len(parent))
    assert (child == exp).all()
    counts, pairs = S.down_rulebook_lists(m, (4096,) * 3, (2048,) * 3)
    o_counts, o_pairs = orc.down2_pairs(parent, off)
    can = orc.canonical_rules(counts.numpy(), pairs.numpy(), o_sc, cc)
    assert (can == orc.canonical_rules(o_counts, o_pairs, o_sc, cc)).all()
    # deconvolution order: a permutation, grouped by offset
    bo = m.deconv_order(fine, d)[:fine.n].cpu().numpy()
    assert (np.sort(bo) == np.arange(fine.n)).all()
    assert (np.diff(off[bo]) >= 0).all()


@pytest.mark.parametrize("P", [3000, 40000])
def test_insert_at_all_scales_equals_the_scale_by_scale_chain(S, P):
    """insc_grid_insert_scales (claim / rank / link at every scale straight from the points) must leave
    the same grids - site ids, coordinates - and the same parent / offset / child links as the chain it
    replaces, insc_grid_insert followed by insc_rulebook_down2 scale by scale; two frames, the second
    with points on old cells, on new cells and repeated, below and above the 16k points one workgroup
    per scale ranks."""
    import ctypes

    from sparseconvnet._lib import InscError, lib, ptr, stream_ptr

    L = 5
    vox = scenes.indoor_scene(seed=61, n=2 * P, dims=(200, 160, 60), n_boxes=12, side_rng=(10, 40)).astype(np.int32)
    rng = np.random.default_rng(61)
    idx2 = np.concatenate([np.arange(P, 2 * P), rng.integers(0, P, P // 8), rng.integers(P, 2 * P, P // 8)])
    frames = [vox[:P], vox[idx2[rng.permutation(len(idx2))]]]
    cap = 4 * P
    vp = ctypes.c_void_p

    def new_grids():
        gs = []
        for _ in range(L):
            g = vp()
            lib.insc_grid_create(I64(cap), ctypes.byref(g))
            gs.append(g)
        par = [torch.full((cap,), -7, dtype=torch.int32, device="cuda") for _ in range(L - 1)]
        off = [torch.full((cap,), -7, dtype=torch.int32, device="cuda") for _ in range(L - 1)]
        chi = [torch.full((cap, 8), -1, dtype=torch.int32, device="cuda") for _ in range(L - 1)]
        return gs, par, off, chi

    def sizes(gs):
        out = []
        for g in gs:
            n = I64(0)
            lib.insc_grid_size(g, ctypes.byref(n), stream_ptr())
            out.append(n.value)
        return out

    # the chain
    ga, pa, oa, ca = new_grids()
    sop_a = []
    for f in frames:
        c = dev(f)
        sop = torch.empty(len(f), dtype=torch.int32, device="cuda")
        before = sizes(ga)
        lib.insc_grid_insert(ga[0], ptr(c), I64(len(f)), ptr(sop), None, stream_ptr())
        after0 = sizes(ga)[0]
        first, n = before[0], after0 - before[0]
        for l in range(L - 1):
            nb = sizes(ga)[l + 1]
            lib.insc_rulebook_down2(ga[l], ga[l + 1], I64(first), I64(n), ptr(pa[l]), ptr(oa[l]), ptr(ca[l]), I64(cap),
                                    stream_ptr())
            first, n = nb, sizes(ga)[l + 1] - nb
        sop_a.append(sop)
    # all scales at once
    gb, pb, ob, cb = new_grids()
    arr = lambda xs: (vp * len(xs))(*[x if isinstance(x, vp) else vp(x.data_ptr()) for x in xs])
    sop_b = []
    counts = (I64 * L)()
    for f in frames:
        c = dev(f)
        sop = torch.empty(len(f), dtype=torch.int32, device="cuda")
        lib.insc_grid_insert_scales(arr(gb), arr(pb + [pb[0]]), arr(ob + [ob[0]]), arr(cb + [cb[0]]), L, ptr(c), 4,
                                    I64(len(f)), ptr(sop), counts, stream_ptr())
        sop_b.append(sop)
    na, nb_ = sizes(ga), sizes(gb)
    assert na == nb_ == list(counts)
    for a, b in zip(sop_a, sop_b):
        assert torch.equal(a, b)
    for l in range(L):
        from sparseconvnet.SCN import _from_ptr

        dv = torch.device("cuda", torch.cuda.current_device())
        ca_ = _from_ptr(lib.insc_grid_coords(ga[l]), (na[l], 4), torch.int32, dv)
        cb_ = _from_ptr(lib.insc_grid_coords(gb[l]), (na[l], 4), torch.int32, dv)
        assert torch.equal(ca_, cb_), "site coordinates of scale %d" % l
        if l + 1 < L:
            assert torch.equal(pa[l][:na[l]], pb[l][:na[l]]), "parents of scale %d" % l
            assert torch.equal(oa[l][:na[l]], ob[l][:na[l]]), "offsets of scale %d" % l
            assert torch.equal(ca[l][:na[l + 1]], cb[l][:na[l + 1]]), "children of scale %d" % (l + 1)
    # a bad coordinate: nothing is inserted anywhere, the grids stay usable
    bad = frames[1].copy()
    bad[7, 2] = 1 << 17
    c = dev(bad)
    sop = torch.empty(len(bad), dtype=torch.int32, device="cuda")
    with pytest.raises(InscError) as e:
        lib.insc_grid_insert_scales(arr(gb), arr(pb + [pb[0]]), arr(ob + [ob[0]]), arr(cb + [cb[0]]), L, ptr(c), 4,
                                    I64(len(bad)), ptr(sop), counts, stream_ptr())
    assert e.value.code == -5
    assert sizes(gb) == na
    for g in ga + gb:
        lib.insc_grid_destroy(g)


def test_orders_of_all_scales_at_once_equal_the_scale_by_scale_calls(S):
    """insc_order_build_scales (the radix passes of all scales in shared launches, inverses written by the
    last pass) against insc_order_build + insc_order_by_offset per scale: the same permutations, word
    for word; three scales of very different size, the last one without a coarser scale above it."""
    import ctypes

    from sparseconvnet._lib import lib, ptr, stream_ptr

    L, P = 3, 60000
    vox = scenes.indoor_scene(seed=77, n=P, dims=(260, 200, 70), n_boxes=15, side_rng=(10, 50)).astype(np.int32)
    cap = 2 * P
    vp = ctypes.c_void_p
    gs = []
    for _ in range(L):
        g = vp()
        lib.insc_grid_create(I64(cap), ctypes.byref(g))
        gs.append(g)
    par = [torch.empty(cap, dtype=torch.int32, device="cuda") for _ in range(L)]
    off = [torch.empty(cap, dtype=torch.int32, device="cuda") for _ in range(L)]
    chi = [torch.full((cap, 8), -1, dtype=torch.int32, device="cuda") for _ in range(L)]
    arr = lambda xs: (vp * len(xs))(*[x if isinstance(x, vp) else vp(x.data_ptr() if x is not None else 0) for x in xs])
    counts = (I64 * L)()
    c = dev(vox)
    sop = torch.empty(P, dtype=torch.int32, device="cuda")
    lib.insc_grid_insert_scales(arr(gs), arr(par), arr(off), arr(chi), L, ptr(c), 4, I64(P), ptr(sop), counts, stream_ptr())
    n = list(counts)
    assert n[0] == P and n[0] > n[1] > n[2] > 8192 // 4
    nbr = [torch.empty((n[l], 27), dtype=torch.int32, device="cuda") for l in range(L)]
    for l in range(L):
        lib.insc_rulebook_ssc3(gs[l], I64(0), I64(n[l]), ptr(nbr[l]), 0, stream_ptr())
    new = lambda l: torch.full((n[l],), -1, dtype=torch.int32, device="cuda")
    # scale by scale
    order_a = [new(l) for l in range(L)]
    bo_a = [new(l) for l in range(L - 1)]
    for l in range(L):
        lib.insc_order_build(gs[l], ptr(nbr[l]), I64(0), I64(n[l]), ptr(order_a[l]), stream_ptr())
        if l + 1 < L:
            lib.insc_order_by_offset(ptr(order_a[l]), ptr(off[l]), I64(n[l]), ptr(bo_a[l]), stream_ptr())
    # all at once
    order_b, pos_b = [new(l) for l in range(L)], [new(l) for l in range(L)]
    bo_b, bop_b = [new(l) for l in range(L)], [new(l) for l in range(L)]
    offs = [off[l] for l in range(L - 1)] + [None]
    lib.insc_order_build_scales(arr(gs), arr(nbr), arr(offs), (I64 * L)(*n), L, arr(order_b), arr(pos_b), arr(bo_b),
                                arr(bop_b), stream_ptr())
    for l in range(L):
        assert torch.equal(order_a[l], order_b[l]), "order of scale %d" % l
        ident = torch.arange(n[l], dtype=torch.int32, device="cuda")
        assert torch.equal(pos_b[l][order_b[l].long()], ident), "inverse of scale %d" % l
        assert torch.equal(torch.sort(order_b[l]).values, ident)
        if l + 1 < L:
            assert torch.equal(bo_a[l], bo_b[l]), "grouped order of scale %d" % l
            assert torch.equal(bop_b[l][bo_b[l].long()], ident), "inverse of the grouped order of scale %d" % l
    assert bool((bo_b[L - 1] == -1).all())  # the scale without a coarser one is left alone
    for g in gs:
        lib.insc_grid_destroy(g)
