"""numpy front end of the CPU oracle (oracle/insc_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the cpu_baseline
leg of the benchmark, never by the shipped package.  Each function is a thin ctypes call
into the C restatement; the reference source each one follows is cited in the C file.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBS = {}
_REAL = np.float32  # arithmetic type of the feature operators: float32 (the reference's) or float64

_i32p = ctypes.POINTER(ctypes.c_int32)


def build(force=False, real=np.float32):
    name = "liborc.so" if real == np.float32 else "liborc64.so"
    so = os.path.join(_HERE, name)
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B", name], stdout=subprocess.DEVNULL)
    return so


def lib():
    if _REAL not in _LIBS:
        L = ctypes.CDLL(build(real=_REAL))
        L.orc_grid_build.restype = ctypes.c_int64
        L.orc_ssc_rules.restype = ctypes.c_int64
        L.orc_down2_rules.restype = ctypes.c_int64
        L.orc_conv_forward.restype = ctypes.c_double
        L.orc_nin_forward.restype = ctypes.c_double
        L.orc_num_threads.restype = ctypes.c_int
        L.orc_real_bytes.restype = ctypes.c_int
        if L.orc_real_bytes() != np.dtype(_REAL).itemsize:
            raise RuntimeError("oracle library built for another arithmetic type")
        _LIBS[_REAL] = L
    return _LIBS[_REAL]


class double_precision(object):
    """`with double_precision():` runs the plain feature operators below (input / output layer,
    rulebook convolution, batch norm, 1x1) through the double-precision build of the same C text
    (liborc64.so): same operations in the same order, no fp32 rounding.  It is the yardstick
    that fp32 results - the oracle's own and the HIP library's - are measured against; the
    residual (incre_*) and pooling operators stay float32."""

    def __enter__(self):
        global _REAL
        self._saved, _REAL = _REAL, np.float64

    def __exit__(self, *exc):
        global _REAL
        _REAL = self._saved


def _ip(a):
    return a.ctypes.data_as(_i32p) if a is not None else None


def _fp(a):
    if a is None:
        return None
    assert a.dtype == _REAL
    return a.ctypes.data_as(ctypes.c_void_p)  # data_as keeps the array alive for the call


def _c4(coords):
    c = np.ascontiguousarray(coords, dtype=np.int32)
    if c.ndim != 2 or c.shape[1] not in (3, 4):
        raise ValueError("coords must be [P,3] or [P,4]")
    if c.shape[1] == 3:
        c = np.concatenate([c, np.zeros((len(c), 1), np.int32)], 1)
    return np.ascontiguousarray(c)


def _f(a):
    return np.ascontiguousarray(a, dtype=_REAL)


def num_threads():
    return lib().orc_num_threads()


def grid_build(coords):
    """-> (site_of_point[P], site_coords[N,4], count[N]); sites numbered by first appearance."""
    c = _c4(coords)
    P = len(c)
    sop = np.empty(P, np.int32)
    sc = np.empty((max(P, 1), 4), np.int32)
    cnt = np.empty(max(P, 1), np.int32)
    n = lib().orc_grid_build(_ip(c), ctypes.c_int64(P), _ip(sop), _ip(sc), _ip(cnt))
    return sop, sc[:n].copy(), cnt[:n].copy()


def grid_query(site_coords, q):
    sc, q = _c4(site_coords), _c4(q)
    out = np.empty(len(q), np.int32)
    lib().orc_grid_query(_ip(sc), ctypes.c_int64(len(sc)), _ip(q), ctypes.c_int64(len(q)), _ip(out))
    return out


def input_forward(feats, site_of_point, count, mode=4):
    f = _f(feats)
    P, C = f.shape
    N = len(count)
    out = np.empty((N, C), _REAL)
    lib().orc_input_forward(_fp(f), ctypes.c_int64(P), C, _ip(np.ascontiguousarray(site_of_point, np.int32)),
                            _ip(np.ascontiguousarray(count, np.int32)), ctypes.c_int64(N), int(mode == 4), _fp(out))
    return out


def output_forward(feats, site_of_point):
    f = _f(feats)
    sop = np.ascontiguousarray(site_of_point, np.int32)
    out = np.empty((len(sop), f.shape[1]), _REAL)
    lib().orc_output_forward(_fp(f), f.shape[1], _ip(sop), ctypes.c_int64(len(sop)), _fp(out))
    return out


def ssc_rules(site_coords, zmajor=False):
    """-> (nbr[N,27], counts[27], pairs[R,2]) ; pairs are the 27 lists back to back."""
    sc = _c4(site_coords)
    N = len(sc)
    nbr = np.empty((N, 27), np.int32)
    counts = np.zeros(27, np.int32)
    pairs = np.empty((max(27 * N, 1), 2), np.int32)
    r = lib().orc_ssc_rules(_ip(sc), ctypes.c_int64(N), int(zmajor), _ip(nbr), _ip(counts), _ip(pairs))
    return nbr, counts, pairs[:r].copy()


def down2_rules(fine_coords):
    """-> (parent[Nf], offset[Nf], coarse_coords[Nc,4])."""
    fc = _c4(fine_coords)
    Nf = len(fc)
    parent = np.empty(Nf, np.int32)
    off = np.empty(Nf, np.int32)
    cc = np.empty((max(Nf, 1), 4), np.int32)
    n = lib().orc_down2_rules(_ip(fc), ctypes.c_int64(Nf), _ip(parent), _ip(off), _ip(cc))
    return parent, off, cc[:n].copy()


def down2_pairs(parent, offset):
    """Rulebook form of a size-2 stride-2 layer: 8 lists of (fine, coarse), back to back."""
    counts = np.bincount(offset, minlength=8).astype(np.int32)
    order = np.argsort(offset, kind="stable")
    pairs = np.stack([order.astype(np.int32), parent[order]], 1)
    return counts, np.ascontiguousarray(pairs, np.int32)


def conv_forward(feats, W, bias, pairs, counts, n_out, swap=False):
    f, W = _f(feats), _f(W)
    K, Cin, Cout = W.shape
    assert f.shape[1] == Cin and len(counts) == K
    out = np.empty((n_out, Cout), _REAL)
    b = _f(bias) if bias is not None else None
    p = np.ascontiguousarray(pairs, np.int32)
    c = np.ascontiguousarray(counts, np.int32)
    flops = lib().orc_conv_forward(_fp(f), _fp(out), ctypes.c_int64(n_out), _fp(W), _fp(b), _ip(p), _ip(c), K, Cin,
                                   Cout, int(swap))
    return out, flops


def bn_forward(feats, mean, var, gamma, beta, eps=1e-4, leakiness=0.0):
    f = _f(feats)
    out = np.empty_like(f)
    g = _f(gamma) if gamma is not None else None
    b = _f(beta) if beta is not None else None
    lib().orc_bn_forward(_fp(f), _fp(out), ctypes.c_int64(f.shape[0]), f.shape[1], _fp(_f(mean)), _fp(_f(var)),
                         _fp(g), _fp(b), ctypes.c_float(eps), ctypes.c_float(leakiness))
    return out


def nin_forward(feats, W, bias=None):
    f, W = _f(feats), _f(W)
    out = np.empty((f.shape[0], W.shape[1]), _REAL)
    b = _f(bias) if bias is not None else None
    lib().orc_nin_forward(_fp(f), _fp(out), ctypes.c_int64(f.shape[0]), _fp(W), _fp(b), W.shape[0], W.shape[1])
    return out


# --------------------------------------------------------------------------------------
# residual frames: the reference's Incre_* operators, restated with numpy.
# A frame has a site set of its own (site_coords of the frame's points); pre_* is the state
# saved by the last full forward.  pre_exist[i] = id of the frame's site i in the saved site
# set, or -1 (getPreExistMaps, Metadata/Metadata.cpp:609-626).
# Pinned in tests/test_oracle_incre.py by the identity every operator must satisfy on its own:
# saved value + residual == the operator applied to the merged scene, at the frame's sites.
# --------------------------------------------------------------------------------------
def incre_pre_exist(pre_coords, coords):
    return grid_query(pre_coords, coords)


def incre_input_forward(feats, site_of_point, count, mode, pre_exist, pre_out, pre_count):
    """InputLayer_inc_fp_ (CUDA/IOLayers.cu:81-105), rule rows as built by inputLayerRules
    (Metadata/IOLayersRules.h:104-129): modes 1/2 keep one row, 3/4 all rows of a voxel."""
    f = _f(feats)
    N, C = len(count), f.shape[1]
    out = np.zeros((N, C), np.float32)
    if mode == 0:  # rows handed through (CUDA/IOLayers.cpp:320-322)
        out[site_of_point] = f
        return out
    rows = [[] for _ in range(N)]
    for p, s in enumerate(site_of_point):
        rows[s].append(p)
    for i in range(N):
        r = rows[i]
        if mode == 1:
            r = r[:1]
        elif mode == 2:
            r = r[-1:]
        pe = int(pre_exist[i])
        na = len(r)
        pn = 0 if pe < 0 else (int(pre_count[pe]) if mode >= 3 else 1)
        m = np.float32(1.0) / np.float32(na + pn) if (mode == 4 and na > 0) else np.float32(1.0)
        acc = np.zeros(C, np.float32)
        for p in r:
            acc = acc + m * f[p]
        if pe >= 0:
            acc = acc + _f(pre_out)[pe] * (np.float32(pn) * m - np.float32(1.0))
        out[i] = acc
    return out


def incre_output_forward(feats, site_of_point, pre_exist, pre_in):
    """InputLayer_inc_bp_ (CUDA/IOLayers.cu:122-141): residual + saved value per point."""
    f, pin = _f(feats), _f(pre_in)
    sop = np.asarray(site_of_point)
    out = f[sop].copy()
    pe = np.asarray(pre_exist)[sop]
    has = pe >= 0
    out[has] += pin[pe[has]]
    return out


def incre_ssc_rules(coords, pre_coords, pre_exist):
    """Rules of IncreSubmanifoldBuildObject (CUDA/SubmanifoldRules_cuda.cpp:233-472): for every
    site of the frame that the saved set does not hold, its 27 neighbours looked up in the saved
    set -> (counts[27], pairs[R,2]) with pairs = (saved site, frame site), the 27 lists back to back."""
    c = _c4(coords)
    new = np.nonzero(np.asarray(pre_exist) < 0)[0]
    counts = np.zeros(27, np.int32)
    lists = []
    for k in range(27):
        d = np.array([k // 9 - 1, (k // 3) % 3 - 1, k % 3 - 1, 0], np.int32)
        q = c[new] + d
        ok = (q[:, :3] >= 0).all(1) & (q[:, :3] < 65536).all(1)
        hit = np.full(len(new), -1, np.int32)
        if ok.any():
            hit[ok] = grid_query(pre_coords, q[ok])
        sel = hit >= 0
        counts[k] = sel.sum()
        lists.append(np.stack([hit[sel], new[sel].astype(np.int32)], 1))
    pairs = np.concatenate(lists, 0) if lists else np.zeros((0, 2), np.int32)
    return counts, np.ascontiguousarray(pairs, np.int32)


def incre_ssc_forward(feats, pre_in, W, bias, rules, rules_pre, n):
    """cuda_Incre_SubmanifoldConvolution_updateOutput (CUDA/Convolution.cpp:221-303): the frame's
    own rules on the residual features, then the rules of incre_ssc_rules on the saved input."""
    out, _ = conv_forward(feats, W, bias, rules[1], rules[0], n)
    if len(rules_pre[1]):
        extra, _ = conv_forward(pre_in, W, None, rules_pre[1], rules_pre[0], n)
        out = out + extra
    return out.astype(np.float32)


def incre_bn_forward(feats, mean, var, gamma, beta, eps, leakiness, pre_exist, pre_in, pre_out):
    """Incre_BatchNormalization_f_test (CUDA/BatchNormalization.cu:112-150)."""
    f = _f(feats)
    C = f.shape[1]
    g = _f(gamma) if gamma is not None else np.ones(C, np.float32)
    bt = _f(beta) if beta is not None else np.zeros(C, np.float32)
    w = (np.power(_f(var) + np.float32(eps), np.float32(-0.5)) * g).astype(np.float32)
    b = (bt - _f(mean) * w).astype(np.float32)
    o = (w * f + b).astype(np.float32)
    pe = np.asarray(pre_exist)
    has = pe >= 0
    t = o.copy()
    t[has] = o[has] + _f(pre_in)[pe[has]] * w
    y = np.where(t > 0, t, t * np.float32(leakiness)).astype(np.float32)
    y[has] -= _f(pre_out)[pe[has]]
    return y


def incre_deconv_forward(feats, pre_in, W, bias, parent, offset, pre_exist_in, pre_exist_out):
    """dDeconvolution_incre_KMxKN_forwardA (CUDA/Deconvolution.cu:84-150): the saved coarse
    feature joins in when the coarse site existed and the fine site is new."""
    f, W = _f(feats), _f(W)
    parent, offset = np.asarray(parent), np.asarray(offset)
    x = f[parent].copy()
    pe_c = np.asarray(pre_exist_in)[parent]
    add = (pe_c >= 0) & (np.asarray(pre_exist_out) < 0)
    x[add] += _f(pre_in)[pe_c[add]]
    out = np.einsum("ni,nio->no", x.astype(np.float64), W[offset].astype(np.float64)).astype(np.float32)
    if bias is not None:
        out = out + _f(bias)
    return out.astype(np.float32)


# --------------------------------------------------------------------------------------
# size-2 stride-2 pooling, unpooling, dense copy (numpy).  Pinned in tests/test_oracle_pool.py
# against torch max_pool3d / avg_pool3d / nearest upsampling on dense tensors and against
# torch.sparse_coo_tensor(...).to_dense().
# --------------------------------------------------------------------------------------
def max_pool_forward(feats, parent, n_coarse, drop=0):
    """MaxPooling_ForwardPass on a zeroed output (CPU/MaxPooling.cpp:7-20, 38-57): max(0, children)."""
    f = _f(feats)[:, drop:]
    out = np.zeros((n_coarse, f.shape[1]), np.float32)
    np.maximum.at(out, np.asarray(parent), f)
    return out


def avg_pool_forward(feats, parent, offset, n_coarse, drop=0):
    """AveragePooling_ForwardPass (CPU/AveragePooling.cpp:7-21): sum over the children of x / 8, the
    rules of offset 0 first, then 1, ... (one pass per offset)."""
    f = _f(feats)[:, drop:]
    out = np.zeros((n_coarse, f.shape[1]), np.float32)
    parent, offset = np.asarray(parent), np.asarray(offset)
    for k in range(8):
        sel = offset == k
        out[parent[sel]] += np.float32(0.125) * f[sel]  # one child per (parent, offset): no repeats
    return out


def unpool_forward(feats, parent, drop=0):
    """UnPooling_ForwardPass (CPU/UnPooling.cpp:7-20): every fine site takes its parent's row."""
    return _f(feats)[:, drop:][np.asarray(parent)].copy()


def sparse_to_dense(feats, site_coords, size, batch):
    """SparseToDense_ForwardPass (CPU/SparseToDense.cpp:7-19): [batch, C, X, Y, Z], zeros elsewhere."""
    f, c = _f(feats), _c4(site_coords)
    out = np.zeros((batch, f.shape[1]) + tuple(size), np.float32)
    out[c[:, 3], :, c[:, 0], c[:, 1], c[:, 2]] = f
    return out


# --------------------------------------------------------------------------------------
# canonical forms used to compare integer structures bit-exactly
# --------------------------------------------------------------------------------------
def canonical_sites(site_coords):
    """Rows sorted by (b, z, y, x): the key order of the reference's GPU grid."""
    sc = _c4(site_coords)
    o = np.lexsort((sc[:, 0], sc[:, 1], sc[:, 2], sc[:, 3]))
    return sc[o]


def canonical_rules(counts, pairs, in_coords, out_coords):
    """Rules as rows (offset, in xyz b, out xyz b), sorted: independent of site numbering."""
    counts = np.asarray(counts)
    k = np.repeat(np.arange(len(counts)), counts).astype(np.int64)
    ic, oc = _c4(in_coords)[pairs[:, 0]].astype(np.int64), _c4(out_coords)[pairs[:, 1]].astype(np.int64)
    rows = np.concatenate([k[:, None], ic, oc], 1)
    o = np.lexsort(tuple(rows[:, j] for j in range(rows.shape[1] - 1, -1, -1)))
    return rows[o]


# ---------------------------------------------------------------------------------------------
# label fusion over frames (Metadata/resultHash.h).  Plain Python over a dict: small cases only.
# ---------------------------------------------------------------------------------------------
class ResultOracle(object):
    """Result<3>::set / update / multiQuery / finalize (resultHash.h:36-145), rows applied one
    after the other.  `maximum` lands in an int member there (resultHash.h:25,30), hence int()."""

    def __init__(self, maximum=0.7):
        self.maximum = int(maximum)
        self.result = {}  # (x,y,z) -> [label, confidence]; insertion order = first appearance

    def set(self, ps, scores):
        for p, row in zip(np.asarray(ps), np.asarray(scores, np.float32)):
            self.result[tuple(int(v) for v in p[:3])] = [int(np.argmax(row)), np.float32(0)]

    def update(self, ps, scores):
        ps, scores = np.asarray(ps), np.asarray(scores, np.float32)
        idx, prob = scores.argmax(1), scores.max(1)  # label.max(1): value and first index
        pre = []
        for p in ps:  # first loop (:62-75): which rows find their voxel already there
            k = tuple(int(v) for v in p[:3])
            pre.append(k in self.result)
            if k not in self.result:
                self.result[k] = [0, np.float32(0)]
        for i, p in enumerate(ps):  # second loop (:78-99)
            e = self.result[tuple(int(v) for v in p[:3])]
            val, mp = int(idx[i]), np.float32(prob[i])
            if not pre[i]:
                e[0], e[1] = val, mp
            else:
                if e[0] == val:
                    e[1] = np.float32(min(np.float32(self.maximum), np.float32(e[1] + mp)))
                else:
                    e[1] = np.float32(e[1] - mp)
                if e[1] < 0:
                    e[0], e[1] = val, np.float32(-e[1])

    def multi_query(self, ps):
        return np.array([self.result.get(tuple(int(v) for v in p[:3]), [-1])[0] for p in np.asarray(ps)], np.int64)

    def finalize(self, points):
        keep = set(tuple(int(v) for v in p[:3]) for p in np.asarray(points))
        self.result = {k: v for k, v in self.result.items() if k in keep}

    def all_points_labels(self):
        return np.array([list(k) + [v[0]] for k, v in self.result.items()], np.int64).reshape(-1, 4)

    def confidences(self):
        return np.array([v[1] for v in self.result.values()], np.float32)


class ResultOfWeightOracle(object):
    """ResultOfWeight::update / multiQuery / finalize (resultHash.h:158-214)."""

    def __init__(self):
        self.result = {}

    def update(self, ps, scores):
        for p, row in zip(np.asarray(ps), np.asarray(scores, np.float32)):
            k = tuple(int(v) for v in p[:3])
            self.result[k] = row.copy() if k not in self.result else (self.result[k] * np.float32(0.5) + row)

    def multi_query(self, ps):
        return np.array([int(np.argmax(self.result[k])) if k in self.result else -1
                         for k in (tuple(int(v) for v in p[:3]) for p in np.asarray(ps))], np.int64)

    def finalize(self, points):
        keep = set(tuple(int(v) for v in p[:3]) for p in np.asarray(points))
        self.result = {k: v for k, v in self.result.items() if k in keep}

    def all_points_labels(self):
        return np.array([list(k) + [int(np.argmax(v))] for k, v in self.result.items()], np.int64).reshape(-1, 4)
