"""msnh_hip_yolo_nms_static -- the device NMS whose workspace is a device array inside the library, for callers that cannot
allocate -- against msnh_hip_yolo_nms with a caller workspace: same record sets, counts and flags, on two calls in a row, the
second on a smaller input (the array keeps the first call's contents).  Both through the kernel C ABI."""
import numpy as np
import pytest
import torch

from msnhnet_amd import hipabi as abi

pytestmark = pytest.mark.gpu


def _rows(rng, batch, cells, classes, crowded):
    """compact candidate rows [batch][cells][8] and counts: objectness / scores on a coarse grid (ties), heavy overlap; image b of
    `crowded` holds that many members of class 0 (more than 1024 takes the large-class kernel, which is the one that uses the workspace)"""
    rows = np.zeros((batch, cells, 8), np.float32)
    cnt = np.zeros(batch, np.int32)
    for b in range(batch):
        n = int(rng.integers(cells // 4, cells // 2))
        r = rows[b, :n]
        r[:, 0:2] = rng.uniform(0, 400, (n, 2))
        r[:, 2:4] = rng.uniform(10, 70, (n, 2))
        r[:, 4] = rng.integers(9, 17, n) / 16.0
        r[:, 5] = rng.integers(1, 9, n) / 8.0
        r[:, 6] = rng.integers(1, classes, n)
        if b in crowded:
            r[:min(n, crowded[b]), 6] = 0
        r[:, 7] = rng.permutation(cells)[:n]
        cnt[b] = n
    return rows, cnt


def _records(kept, kc):
    rec = kept[:int(kc[0])]
    return rec[np.lexsort(rec.T[::-1])]


def _both(batch, classes, cells, rows, cnt, thr):
    import gpuutil as gu
    L = abi.lib()
    rd, cd = gu.dev(rows), gu.dev(cnt)
    nbytes = L.msnh_hip_yolo_nms_workspace_bytes(batch, classes, cells)
    out = []
    for static in (False, True):
        kept = torch.zeros((batch * cells, 12), dtype=torch.float32).cuda()
        kc = torch.zeros(1 + batch, dtype=torch.int32).cuda()
        ws = torch.full((nbytes // 4,), 0x55555555, dtype=torch.int32).cuda()
        gu.sync()
        if static:
            abi.check(L.msnh_hip_yolo_nms_static(batch, classes, gu.ptr(rd), cells, gu.ptr(cd), thr, gu.ptr(kept), batch * cells, gu.ptr(kc), None))
        else:
            abi.check(L.msnh_hip_yolo_nms(batch, classes, gu.ptr(rd), cells, gu.ptr(cd), thr, gu.ptr(kept), batch * cells, gu.ptr(kc), gu.ptr(ws), nbytes, None))
        gu.sync()
        out.append((kept.cpu().numpy(), kc.cpu().numpy()))
    return out


def test_yolo_nms_static_equals_workspace_variant():
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    assert L.msnh_hip_yolo_nms_static_max_bytes() == 4 << 20
    rng = np.random.default_rng(77)
    classes, thr = 6, 0.45
    # first call: 5 images of 6912 slots, two of them with a class of 1500 / 3000 members; second call: 2 images of 2000 slots, one crowded
    for batch, cells, crowded in ((5, 6912, {1: 1500, 3: 3000}), (2, 3000, {0: 1100})):
        rows, cnt = _rows(rng, batch, cells, classes, crowded)
        print("yolo_nms_static", batch, cells, cnt.tolist(), flush=True)
        (kept_a, kc_a), (kept_b, kc_b) = _both(batch, classes, cells, rows, cnt, thr)
        assert np.array_equal(kc_a, kc_b), (kc_a, kc_b)
        assert kc_a[0] > 0 and not kc_a[1:].any()
        assert np.array_equal(_records(kept_a, kc_a), _records(kept_b, kc_b))
    # beyond the built-in workspace: refused with a message, nothing launched
    kc = torch.zeros(65, dtype=torch.int32).cuda()
    rd = torch.zeros(16, dtype=torch.float32).cuda()
    assert L.msnh_hip_yolo_nms_static(64, 80, gu.ptr(rd), 22743, gu.ptr(kc), thr, gu.ptr(rd), 64 * 22743, gu.ptr(kc), None) != 0
    assert b"built-in one holds" in L.msnh_hip_last_error()


def test_yolo_nms_static_calls_on_two_streams_are_put_in_order():
    """two calls issued back to back on two different streams, and two calls from two host threads, all on the one built-in workspace:
    the library makes each wait for the one before it on the device, so every result equals the caller-workspace variant's"""
    import ctypes
    import threading
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    rng = np.random.default_rng(78)
    classes, thr = 6, 0.45
    cases = []
    for batch, cells, crowded in ((4, 6912, {0: 2500, 2: 1800}), (3, 4000, {1: 1300}), (4, 6912, {3: 3000}), (2, 3000, {0: 1100})):
        rows, cnt = _rows(rng, batch, cells, classes, crowded)
        (kept_a, kc_a), _ = _both(batch, classes, cells, rows, cnt, thr)
        cases.append((batch, cells, gu.dev(rows), gu.dev(cnt), _records(kept_a, kc_a), kc_a))
    streams = []
    for _ in range(2):
        s = ctypes.c_void_p()
        abi.check(L.msnh_hip_stream_create(ctypes.byref(s)))
        streams.append(s)
    outs = [(torch.zeros((b * c, 12), dtype=torch.float32).cuda(), torch.zeros(1 + b, dtype=torch.int32).cuda()) for b, c, *_ in cases]
    gu.sync()

    def call(i, stream):
        b, c, rd, cd, _, _ = cases[i]
        kept, kc = outs[i]
        abi.check(L.msnh_hip_yolo_nms_static(b, classes, gu.ptr(rd), c, gu.ptr(cd), thr, gu.ptr(kept), b * c, gu.ptr(kc), stream))

    print("yolo_nms_static on two streams", flush=True)
    call(0, streams[0])
    call(1, streams[1])                 # enqueued while the first may still run: waits for it on the device
    threads = [threading.Thread(target=call, args=(2, streams[0])), threading.Thread(target=call, args=(3, streams[1]))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for s in streams:
        abi.check(L.msnh_hip_stream_sync(s))
    for i, (b, c, rd, cd, want, want_kc) in enumerate(cases):
        kept, kc = outs[i][0].cpu().numpy(), outs[i][1].cpu().numpy()
        assert np.array_equal(kc, want_kc), (i, kc, want_kc)
        assert np.array_equal(_records(kept, kc), want), i
    for s in streams:
        abi.check(L.msnh_hip_stream_destroy(s))
