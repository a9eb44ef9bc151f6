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


def thresholds(arch):
    """(confThresh, nmsThresh) the generated graph of a detector carries"""
    import inspect
    sig = inspect.signature(zoo.ARCHS[arch]).parameters
    return float(sig["conf"].default), float(sig["nms"].default)


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


# ---- detection candidates cell by cell ----------------------------------------------------------------------------------------------
def yolo_scan(decoded_heads, per, conf_thresh):
    """the reference's candidate scan (src/layers/MsnhYoloOutLayer.cpp:120-170) over decoded head tensors, each flat [3*per, H*W]:
    rows [n, 8] = x y w h objectness, best class score, first-maximum class, cell number, in scan order (cells ascending: head by
    head, anchor, pixel); the test is objectness > conf_thresh on the decoded value"""
    rows, base = [], 0
    for d in decoded_heads:
        hw = d.size // (3 * per)
        v = np.asarray(d, np.float32).reshape(3, per, hw).transpose(0, 2, 1).reshape(3 * hw, per)
        c = np.nonzero(v[:, 4] > conf_thresh)[0]
        r = np.zeros((len(c), 8), np.float32)
        r[:, :5] = v[c, :5]
        if len(c):
            r[:, 5] = v[c, 5:].max(1)
            r[:, 6] = v[c, 5:].argmax(1)
        r[:, 7] = c + base
        rows.append(r)
        base += 3 * hw
    return np.concatenate(rows) if rows else np.zeros((0, 8), np.float32)


def head_logits_by_cell(logit_heads, per):
    """head logit tensors (each flat [3*per, H*W], NCHW) -> [cells, per] in the scan's cell order, and the head of every cell"""
    out, head = [], []
    for k, t in enumerate(logit_heads):
        hw = t.size // (3 * per)
        out.append(np.asarray(t, np.float64).reshape(3, per, hw).transpose(0, 2, 1).reshape(3 * hw, per))
        head.append(np.full(3 * hw, k, np.int64))
    return np.concatenate(out), np.concatenate(head)


def same_box_set(a, b):
    """two sets of 7-float boxes are the same multiset, bit for bit (NaN equal to NaN)"""
    a, b = sort_boxes(a), sort_boxes(b)
    return a.shape == b.shape and np.array_equal(a, b, equal_nan=True)


def attribute_candidates(dev_rows, ref_rows, near, tol=2e-2):
    """Compares the candidate rows of the device with the reference's, cell by cell.

    dev_rows, ref_rows: [n, 8] rows as yolo_scan returns them (any order).  near(cells, channel) -> bool array: whether the reference's
    logit of that cell and channel (0 x, 1 y, 2 w, 3 h, 4 objectness, 5+j class j) lies within the float16 logit error of a point where
    the decoded value jumps (zero for the logistic outputs, the range where exp is finite for w and h).

    Returns (only_dev, only_ref, differing, unexplained): cells that are a candidate on one side only, common cells whose rows differ
    (a finite column beyond tol * max|reference column|, another inf / NaN pattern, another class), and a list of descriptions of every
    difference that `near` does not explain -- empty when every difference is attributed to a logit next to a decision point."""
    dev_rows = np.asarray(dev_rows, np.float32).reshape(-1, 8)
    ref_rows = np.asarray(ref_rows, np.float32).reshape(-1, 8)
    dcell, rcell = dev_rows[:, 7].astype(np.int64), ref_rows[:, 7].astype(np.int64)
    assert len(np.unique(dcell)) == len(dcell) and len(np.unique(rcell)) == len(rcell), "a cell appears twice"
    only_dev = np.setdiff1d(dcell, rcell)
    only_ref = np.setdiff1d(rcell, dcell)
    unexplained = []
    for cells, side in ((only_dev, "device only"), (only_ref, "reference only")):
        if len(cells):
            ok = near(cells, np.full(len(cells), 4))
            unexplained += [f"cell {c}: candidate on the {side}, objectness logit not near zero" for c in cells[~ok]]
    common, di, ri = np.intersect1d(dcell, rcell, return_indices=True)
    d, r = dev_rows[di].astype(np.float64), ref_rows[ri].astype(np.float64)
    differing = np.zeros(len(common), bool)
    for col in range(6):
        chan = np.full(len(common), col) if col < 5 else 5 + r[:, 6].astype(np.int64)
        fin = np.isfinite(r[:, col])
        scale = max(np.abs(r[fin, col]).max(), 1e-30) if fin.any() else 1.0
        with np.errstate(invalid="ignore"):
            bad = np.where(fin, ~(np.abs(d[:, col] - r[:, col]) <= tol * scale), ~((d[:, col] == r[:, col]) | (np.isnan(d[:, col]) & np.isnan(r[:, col]))))
        bad &= d[:, 6] == r[:, 6]              # (rows of another class are handled below: their class score belongs to another channel)
        if bad.any():
            ok = near(common[bad], chan[bad])
            unexplained += [f"cell {c} column {col}: {a} vs {b}" for c, a, b in zip(common[bad][~ok], d[bad][~ok, col], r[bad][~ok, col])]
            differing |= bad
    cls_bad = d[:, 6] != r[:, 6]
    for i in np.nonzero(cls_bad)[0]:
        # first-maximum class: it can only move if a class up to the later of the two has a logit next to zero (scores saturate at 1)
        hi = int(max(d[i, 6], r[i, 6]))
        if not near(np.full(hi + 1, common[i]), 5 + np.arange(hi + 1)).any():
            unexplained.append(f"cell {common[i]}: class {int(d[i, 6])} vs {int(r[i, 6])}")
    differing |= cls_bad
    return only_dev, only_ref, common[differing], unexplained


def attribute_against_reference(dev_rows, dev_logit_heads, ref_decoded_heads, ref_logit_heads, per, conf_thresh, bar=2e-2):
    """The float16 candidates of one image against the reference's, every difference attributed.

    dev_rows: candidate rows of the device [n, 8]; dev_logit_heads / ref_logit_heads: per head the logit tensor of this image (flat NCHW);
    ref_decoded_heads: the reference's decoded head tensors.  Checks that the measured logit error of every head is within
    bar * max|reference logits| and that every candidate-set or row difference sits on a reference logit no farther from a jump of the
    decode than that head's measured error (+ 90: the width of the range where exp() is finite and the logistic is not yet exactly 0 or 1).
    Returns (ref_rows, only_dev, only_ref, differing_cells, head_errors)."""
    ref_rows = yolo_scan(ref_decoded_heads, per, conf_thresh)
    ref_l, head = head_logits_by_cell(ref_logit_heads, per)
    dev_l, _ = head_logits_by_cell(dev_logit_heads, per)
    assert ref_l.shape == dev_l.shape
    fin = np.isfinite(ref_l)
    assert (np.isfinite(dev_l) == fin).all()
    err = np.zeros(len(ref_logit_heads))
    for k in range(len(ref_logit_heads)):
        sel = head == k
        d = np.abs(np.where(fin[sel], dev_l[sel] - ref_l[sel], 0.0))
        err[k] = d.max()
        assert err[k] <= bar * np.abs(ref_l[sel][fin[sel]]).max(), (k, err[k])

    def near(cells, chans):
        return np.abs(ref_l[cells, chans]) <= err[head[cells]] + 90.0

    only_dev, only_ref, differing, unexplained = attribute_candidates(dev_rows, ref_rows, near, bar)
    assert not unexplained, unexplained[:10]
    # a cell that is a candidate on one side only: the two objectness logits lie on opposite sides of the threshold, so the
    # reference's is no farther from it than the two are apart
    for cells in (only_dev, only_ref):
        if len(cells):
            assert (np.abs(ref_l[cells, 4]) <= np.abs(dev_l[cells, 4] - ref_l[cells, 4]) + 1e-3).all()
    return ref_rows, only_dev, only_ref, differing, err


def _iou_plus1(a, b):
    """Box::iou with the reference's +1 extents (include/Msnhnet/utils/MsnhTypes.h:123-140) on rows x y w h"""
    ax1, ax2, ay1, ay2 = a[0] - a[2] / 2, a[0] + a[2] / 2, a[1] - a[3] / 2, a[1] + a[3] / 2
    bx1, bx2, by1, by2 = b[0] - b[2] / 2, b[0] + b[2] / 2, b[1] - b[3] / 2, b[1] + b[3] / 2
    iw = max(min(ax2, bx2) - max(ax1, bx1) + 1, 0.0)
    ih = max(min(ay2, by2) - max(ay1, by1) + 1, 0.0)
    inter = iw * ih
    return inter / ((ax2 - ax1 + 1) * (ay2 - ay1 + 1) + (bx2 - bx1 + 1) * (by2 - by1 + 1) - inter)


def box_sets_equal_up_to_ties(got, ref, nms_thresh):
    """Two NMS results over the same candidates are the same multiset of boxes bit for bit, except where the reference's own result is
    not determined by its input: it orders the candidates with std::sort (include/Msnhnet/utils/MsnhExVector.h:57-74), which leaves the
    order of candidates with equal objectness * class score unspecified, and among candidates of equal objectness the greedy loop keeps
    whichever comes first.  A box present on one side only must therefore have a partner on the other side only with the same class,
    objectness and class score that it overlaps by more than the threshold (either suppresses the other).  Returns the number of such
    swapped pairs; raises AssertionError otherwise."""
    got = np.asarray(got, np.float32).reshape(-1, 7)
    ref = np.asarray(ref, np.float32).reshape(-1, 7)
    assert len(got) == len(ref), (len(got), len(ref))
    key = lambda r: tuple(np.nan_to_num(r.astype(np.float64), nan=-7e300).tolist())
    from collections import Counter
    cg, cr = Counter(key(r) for r in got), Counter(key(r) for r in ref)
    only_g, only_r = list((cg - cr).elements()), list((cr - cg).elements())
    assert len(only_g) == len(only_r)
    for a in only_g:
        j = next((j for j, b in enumerate(only_r) if a[4:7] == b[4:7] and _iou_plus1(a, b) > nms_thresh), None)
        assert j is not None, f"box {a} has no tied, overlapping partner among {only_r[:5]}"
        only_r.pop(j)
    return len(only_g)
