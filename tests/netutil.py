"""Shared helpers of the network-level tests: model files in a temp dir, reference / oracle runs, comparisons."""
import os
import tempfile

import numpy as np

from msnhnet_amd import zoo

_dir = None


def workdir():
    global _dir
    if _dir is None:
        _dir = tempfile.mkdtemp(prefix="msnh_models_")
    return _dir


def model(arch, batch, size, seed=1, **kw):
    """Writes graph + seeded weights once per (arch,batch,size,seed); returns (msnhnet, msnhbin, GraphWriter)."""
    net, binp, g = zoo.write_model(arch, workdir(), batch, size, seed=seed, **kw)
    return net, binp, g


def batch1_graph(arch, size, **kw):
    g = zoo.ARCHS[arch](batch=1, size=size, **kw)
    path = os.path.join(workdir(), f"{arch}_b1_{size}_oracle.msnhnet")
    with open(path, "w") as f:
        f.write(g.text())
    return path


def facade_shuffle(pre, swap_rgb):
    """whether the network behind the reference's C facade (the build without OpenCV) sees the first and third channel of the caller's
    image exchanged: the facade exchanges them when swapRGB == 0 (src/c_api/MsnhnetLib.cpp:562, :771), CVUtil's default needShuffleRGB
    (include/Msnhnet/utils/MsnhCVUtil.h:23-38) exchanges them again for every form but the letterbox.  tests/test_ref_facade_cpu.py
    checks this table against the reference's facade itself."""
    return (not swap_rgb) if pre == "padding_zero" else bool(swap_rgb)


def rel_err(a, b):
    """max|a-b|/max|b| over entries finite in the reference; non-finite entries must agree in class and sign."""
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    assert a.shape == b.shape, (a.shape, b.shape)
    fb = np.isfinite(b)
    bad = ~fb
    if bad.any():
        assert (np.isnan(a[bad]) == np.isnan(b[bad])).all(), "NaN pattern differs"
        inf = bad & ~np.isnan(b)
        assert (a[inf] == b[inf]).all(), "inf pattern differs"
    if not fb.any():
        return 0.0
    assert np.isfinite(a[fb]).all(), "non-finite value where the reference is finite"
    return float(np.abs(a[fb] - b[fb]).max() / max(np.abs(b[fb]).max(), 1e-30))


def sort_boxes(b):
    b = np.asarray(b, np.float32).reshape(-1, 7)
    if len(b) == 0:
        return b
    key = np.nan_to_num(b, nan=1e30, posinf=2e30, neginf=-2e30)
    return b[np.lexsort(key.T[::-1])]


def _box_embedding(b):
    """rows of 7 floats -> points whose Euclidean neighbours are the boxes that nearly equal them (sizes on a log scale: they
    overflow to inf with the seeded weights; the class index far apart)"""
    k = np.asarray(b, np.float64).reshape(-1, 7).copy()
    wh = k[:, 2:4]
    wh = np.where(np.isnan(wh), 400.0, np.sign(wh) * np.log1p(np.minimum(np.abs(wh), 1e300)))
    k[:, 2:4] = np.where(np.isinf(k[:, 2:4]), np.sign(k[:, 2:4]) * 800.0, wh)
    k[:, 0:2] = np.nan_to_num(k[:, 0:2], nan=1e6, posinf=2e6, neginf=-2e6)
    k[:, 4:6] = np.nan_to_num(k[:, 4:6], nan=50.0) * 100.0
    k[:, 6] *= 1e4
    return k


def boxes_one_sided_err(sub, full):
    """every box of `sub` has a box of `full` next to it: returns the largest column-wise deviation |sub - nearest| / max|full| over the
    finite entries (non-finite entries and the class index must agree exactly).  Unlike a comparison of two sorted lists this does not
    depend on how boxes that differ in the last bits are ordered."""
    from scipy.spatial import cKDTree
    sub = np.asarray(sub, np.float32).reshape(-1, 7)
    full = np.asarray(full, np.float32).reshape(-1, 7)
    if len(sub) == 0:
        return 0.0
    assert len(full) > 0, "no boxes to match against"
    _, idx = cKDTree(_box_embedding(full)).query(_box_embedding(sub))
    near = full[idx]
    assert np.array_equal(sub[:, 6], near[:, 6]), "class of the nearest box differs"
    return rel_err(sub[:, :6], near[:, :6])


def boxes_matched_fraction(got, ref, tol):
    """fraction of the boxes of `got` that have a box of `ref` of the same class within tol * max|ref| in every finite column.  For
    comparisons across two builds of a plan: with the seeded weights most objectness values saturate at exactly 1, suppression among
    such ties depends on the last bit of the few values that do not, and two tile choices differ in exactly those bits -- so a few
    boxes of a crowded image may legitimately be replaced by their neighbours."""
    from scipy.spatial import cKDTree
    got = np.asarray(got, np.float32).reshape(-1, 7)
    ref = np.asarray(ref, np.float32).reshape(-1, 7)
    if len(got) == 0 or len(ref) == 0:
        return 1.0 if len(got) == len(ref) else 0.0
    _, idx = cKDTree(_box_embedding(ref)).query(_box_embedding(got))
    near = ref[idx].astype(np.float64)
    g = got.astype(np.float64)
    fin = np.isfinite(near[:, :6])
    scale = max(np.abs(near[:, :6][fin]).max(), 1e-30) if fin.any() else 1.0
    with np.errstate(invalid="ignore"):
        ok_fin = np.where(fin, np.abs(g[:, :6] - near[:, :6]) <= tol * scale, True)
        ok_inf = np.where(fin, True, (g[:, :6] == near[:, :6]) | (np.isnan(g[:, :6]) & np.isnan(near[:, :6])))
    ok = ok_fin.all(1) & ok_inf.all(1) & (g[:, 6] == near[:, 6])
    return float(ok.mean())


def boxes_err(got, ref):
    """two box sets agree: same count, and each box of either set has a box of the other next to it (see boxes_one_sided_err)"""
    got = np.asarray(got, np.float32).reshape(-1, 7)
    ref = np.asarray(ref, np.float32).reshape(-1, 7)
    assert len(got) == len(ref), f"box count {len(got)} vs {len(ref)}"
    return max(boxes_one_sided_err(got, ref), boxes_one_sided_err(ref, got))


def yolo_layer_err(got, ref, logits, channels_per_anchor, ratio, version=3):
    """Error of a decoded yolo layer [3*per, H*W] in units of the logit error that explains it.

    Every decoded value is a function of one logit t: (sigmoid(t)+cell)*ratio, anchor*exp(t) or sigmoid(t).  A logit
    error d (itself bounded relative to max|t|) shows up as at most d/4 in a sigmoid plane and as a factor e^d in a
    w,h plane, however small d/|t| is.  So: sigmoid planes -> absolute error (x,y divided by ratio), w,h planes ->
    |log got - log ref|, all divided by max(1, max|t|).  yolov5 (version 5) decodes with 2*sigmoid and (2*sigmoid)^2: its
    x,y and w,h errors are twice as sensitive, and a squared sigmoid underflows gradually instead of overflowing."""
    per = channels_per_anchor
    got = np.asarray(got, np.float64).reshape(3, per, -1)
    ref = np.asarray(ref, np.float64).reshape(3, per, -1)
    scale = max(np.abs(np.asarray(logits, np.float64)).max(), 1.0)
    e_xy = np.abs(got[:, 0:2] - ref[:, 0:2]).max() / ratio
    e_sig = np.abs(got[:, 4:] - ref[:, 4:]).max()
    g, r = got[:, 2:4].ravel(), ref[:, 2:4].ravel()
    fin = np.isfinite(r) & (r != 0)
    if version == 5:
        tiny = 1e-30                      # (2*sigmoid)^2 below this is in or next to the subnormal range: only require both to be tiny
        assert np.isfinite(g).all() and np.isfinite(r).all() and (np.abs(g[np.abs(r) < tiny]) < 1e-25).all() and (np.abs(r[np.abs(g) < tiny]) < 1e-25).all()
        fin = (np.abs(r) >= tiny) & (np.abs(g) >= tiny)
        e_xy /= 2.0
    else:
        assert (np.isfinite(g) == np.isfinite(r)).all() and ((g == 0) == (r == 0)).all(), "inf / underflow pattern differs"
    e_wh = float(np.abs(np.log(np.abs(g[fin])) - np.log(np.abs(r[fin]))).max()) if fin.any() else 0.0
    if version == 5:
        e_wh /= 2.0
    return float(max(e_xy, e_sig, e_wh) / scale)


def layer_stats(a):
    """the 22 numbers the golden files keep per layer output: size, finite count, sum, abs-sum, max, min, 16 sampled values"""
    a = np.asarray(a, np.float64).ravel()
    fin = np.isfinite(a)
    v = a[fin]
    idx = (np.arange(16) * 7919) % max(a.size, 1)
    return np.array([a.size, fin.sum(), v.sum() if v.size else 0, np.abs(v).sum() if v.size else 0, v.max() if v.size else 0,
                     v.min() if v.size else 0] + [a[i] if a.size else 0 for i in idx], np.float64)


def stats_err(got, want):
    """layer statistics against stored ones, relative to the layer's range (sums relative to the abs-sum)"""
    size, nfin, s, sabs, mx, mn = want[:6]
    assert got[0] == size and got[1] == nfin, ("element / finite count differs", got[:2], want[:2])
    rng = max(abs(mx), abs(mn), 1e-30)
    e = max(abs(got[4] - mx), abs(got[5] - mn)) / rng
    e = max(e, abs(got[2] - s) / max(sabs, 1e-30), abs(got[3] - sabs) / max(sabs, 1e-30))
    ok = np.isfinite(want[6:])
    if ok.any():
        e = max(e, float(np.abs(got[6:][ok] - want[6:][ok]).max()) / rng)
    return float(e)
