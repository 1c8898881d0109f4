#!/usr/bin/env python3
"""Times every operator of the library on the five reference workloads.

  python -m vkop_amd.bench_ops [--steps K] [--warmup W] [--only NAME_SUBSTRING] [--eager]
  python -m vkop_amd.bench_ops --data-sweep [--only NAME_SUBSTRING]
  python -m vkop_amd.bench_ops --softmax-sweep [--only NAME_SUBSTRING]

bench.py at the repository root measures the headline (fused softmax -> top-k on
[64,128256]); this script covers the rest: plain softmax, plain top-k, the fused
operator and the detection-style chain on all five workloads, one call in flight,
K calls recorded once and replayed, HIP events around the replay.  Inputs rotate
over enough device buffers (> 288 MB) that the Infinity Cache cannot serve them.
Prints one JSON line per case: microseconds per call and the algorithmic rate
(compulsory reads + final writes over time).

--data-sweep instead times top-k (largest, smallest) and the fused call on a dozen
shapes x fourteen kinds of rows (sorted, constant, two values, a dozen levels, masked,
NaN / +inf rows, one value with peaks, sorted runs, ...) in single and half precision and
flags every case that takes more than three times the same shape's normal rows: the
places where a selection kernel falls off a cliff.

--softmax-sweep times the plain softmax on two dozen shapes (short rows by the ten
thousand, attention-shaped tensors, the workloads' shapes, rows of a million, lines along
a non-last axis short and long) in single and half precision against the bytes moved.
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--only", default="")
    ap.add_argument("--data-sweep", action="store_true",
                    help="time top-k and the fused call on shapes x kinds of awkward rows instead of the workloads")
    ap.add_argument("--softmax-sweep", action="store_true", help="time the plain softmax on a range of shapes and axes")
    ap.add_argument("--eager", action="store_true",
                    help="launch every call from the host instead of replaying a recording (for counter runs under "
                         "rocprofv3 --pmc; the timings of such a run mean nothing)")
    args = ap.parse_args()

    import numpy as np
    import torch

    from vkop_amd import capi, synth

    capi.init(0)
    stream = capi.stream_create()
    e0, e1 = capi.event_create(), capi.event_create()
    F32, F16 = capi.F32, capi.F16

    def buffers(x):
        nbuf = min(64, max(2, -(-(288 << 20) // x.nbytes)))
        return [torch.from_numpy(x).cuda() for _ in range(nbuf)]

    def workspace(nbytes):
        ws = torch.empty(nbytes + 256, dtype=torch.uint8, device="cuda")
        ptr = ws.data_ptr() + (-ws.data_ptr()) % 256
        capi.workspace_init(ptr, nbytes // 4 * 4, stream)
        capi.stream_sync(stream)
        return ws, ptr

    def timed(call, nbuf):
        if args.eager:
            for i in range(args.warmup + args.steps):
                call(i % nbuf)
            capi.stream_sync(stream)
            return None

        def record(count, first):
            capi.graph_begin(stream)
            for i in range(first, first + count):
                call(i % nbuf)
            return capi.graph_end(stream)
        gw = record(args.warmup, 0)
        capi.graph_launch(gw, stream)
        gk = record(args.steps, args.warmup)
        capi.stream_sync(stream)
        capi.event_record(e0, stream)
        capi.graph_launch(gk, stream)
        capi.event_record(e1, stream)
        capi.event_sync(e1)
        ms = capi.event_elapsed_ms(e0, e1)
        capi.graph_destroy(gw)
        capi.graph_destroy(gk)
        return ms / args.steps * 1e3

    def report(name, us, algo_bytes):
        if us is None:
            print(json.dumps({"case": name, "eager": True, "algorithmic_bytes": algo_bytes}), flush=True)
            return
        print(json.dumps({"case": name, "us_per_call": round(us, 2), "algorithmic_bytes": algo_bytes,
                          "algorithmic_GBps": round(algo_bytes / us / 1e3, 1),
                          "frac_of_8TBps": round(algo_bytes / us / 1e3 / 8000.0, 4)}), flush=True)

    def softmax_case(name, x, axis):
        if args.only not in name:
            return
        dt = F16 if x.dtype == np.float16 else F32
        bufs = buffers(x.view(np.uint16) if dt == F16 else x)
        out = torch.empty_like(bufs[0])
        nb = capi.softmax_workspace_bytes(dt, x.shape, axis)
        ws, ptr = workspace(nb + 256)
        us = timed(lambda b: capi.softmax(bufs[b].data_ptr(), out.data_ptr(), dt, x.shape, axis, 0, 0.0, ptr, nb + 256,
                                          stream), len(bufs))
        report(name, us, 2 * x.nbytes)

    def select_case(name, x, k, fused, largest=1, sorted_=1):
        if args.only not in name:
            return
        dt = F16 if x.dtype == np.float16 else F32
        bufs = buffers(x.view(np.uint16) if dt == F16 else x)
        rows = int(np.prod(x.shape[:-1]))
        vals = torch.empty((rows, k), dtype=bufs[0].dtype, device="cuda")
        idx = torch.empty((rows, k), dtype=torch.int32, device="cuda")
        nb = (capi.softmax_topk_workspace_bytes if fused else capi.topk_workspace_bytes)(dt, x.shape, -1, k)
        ws, ptr = workspace(nb + 256)
        if fused:
            call = lambda b: capi.softmax_topk(bufs[b].data_ptr(), 0, vals.data_ptr(), idx.data_ptr(), dt, x.shape, -1, k,
                                               1, ptr, nb + 256, stream)
        else:
            call = lambda b: capi.topk(bufs[b].data_ptr(), vals.data_ptr(), idx.data_ptr(), dt, x.shape, -1, k, largest, sorted_,
                                       ptr, nb + 256, stream)
        us = timed(call, len(bufs))
        report(name, us, x.nbytes + rows * k * (x.itemsize + 4))

    def sampling_case(name, x, k, scale, top_p):
        """vkop_hip_softmax_topk_sampling: temperature and nucleus count inside the call."""
        if args.only not in name:
            return
        bufs = buffers(x)
        rows = int(np.prod(x.shape[:-1]))
        vals = torch.empty((rows, k), dtype=bufs[0].dtype, device="cuda")
        idx = torch.empty((rows, k), dtype=torch.int32, device="cuda")
        counts = torch.empty((rows,), dtype=torch.int32, device="cuda")
        nb = capi.softmax_topk_workspace_bytes(F32, x.shape, -1, k)
        ws, ptr = workspace(nb + 256)
        us = timed(lambda b: capi.softmax_topk_sampling(bufs[b].data_ptr(), vals.data_ptr(), idx.data_ptr(), counts.data_ptr(), F32,
                                                        x.shape, -1, k, scale, top_p, ptr, nb + 256, stream), len(bufs))
        report(name, us, x.nbytes + rows * (k * (x.itemsize + 4) + 4))

    if args.softmax_sweep:
        shapes = [((256, 1000), -1), ((4096, 32), -1), ((65536, 64), -1), ((16384, 128), -1), ((8192, 256), -1), ((4096, 1024), -1),
                  ((2048, 2048), -1), ((1024, 4096), -1), ((256, 8192), -1), ((128, 16384), -1), ((64, 32768), -1), ((32, 50257), -1),
                  ((64, 128256), -1), ((8, 262144), -1), ((4, 1048576), -1), ((128, 12, 197, 197), -1), ((16, 32, 1024, 1024), -1),
                  ((16, 80, 8400), 1), ((64, 8, 4096), 1), ((8, 21, 512, 512), 1), ((32, 1000, 64), 1), ((8, 4096, 256), 1),
                  ((1, 4096, 4096), 1)]
        rng = np.random.default_rng(3)
        for shape, axis in shapes:
            for dt, tdt, dname in ((F32, torch.float32, "f32"), (F16, torch.float16, "f16")):
                name = "softmax %s axis %d %s" % (list(shape), axis, dname)
                if args.only not in name:
                    continue
                x = (rng.standard_normal(shape, dtype=np.float32) * np.float32(1.25))
                nb = max(2, min(16, (300 << 20) // (x.nbytes if dt == F32 else x.nbytes // 2)))
                bufs = [torch.from_numpy(x).cuda().to(tdt) for _ in range(nb)]
                out = torch.empty_like(bufs[0])
                wsb = capi.softmax_workspace_bytes(dt, shape, axis)
                ws, ptr = workspace(wsb + 256)
                us = timed(lambda b: capi.softmax(bufs[b].data_ptr(), out.data_ptr(), dt, shape, axis, 0, 0.0, ptr, wsb + 256, stream), nb)
                report(name, us, 2 * bufs[0].numel() * bufs[0].element_size())
        return

    if args.data_sweep:
        shapes = [(256, 1000, 5), (8192, 256, 8), (4096, 1024, 32), (1024, 4096, 64), (256, 8192, 100), (16, 8400, 300),
                  (64, 32000, 40), (32, 50257, 200), (64, 128256, 50), (16, 100000, 600), (8, 262144, 1024), (8, 262144, 2000),
                  (4, 1048576, 100)]
        for rows, n, k in shapes:
            for dt, tdt, dname in ((F32, torch.float32, "f32"), (F16, torch.float16, "f16")):
                base = None
                names = {kind: "[%d,%d] k=%d %s %s" % (rows, n, k, dname, kind) for kind in synth.AWKWARD_KINDS}
                if not any(args.only in nm for nm in names.values()):
                    continue
                for kind in synth.AWKWARD_KINDS:
                    name = names[kind]
                    if args.only not in name and kind != "normal":  # (the normal rows are every case's yardstick)
                        continue
                    x = synth.awkward_rows(kind, rows, n, seed=rows + n + k)
                    nb = max(2, min(16, (64 << 20) // x.nbytes))
                    bufs = [torch.from_numpy(x).cuda().to(tdt) for _ in range(nb)]
                    vals = torch.empty((rows, k), dtype=tdt, device="cuda")
                    idx = torch.empty((rows, k), dtype=torch.int32, device="cuda")
                    wsb = max(capi.topk_workspace_bytes(dt, (rows, n), -1, k), capi.softmax_topk_workspace_bytes(dt, (rows, n), -1, k))
                    ws, ptr = workspace(wsb + 256)
                    sh = (rows, n)
                    us = [timed(lambda b: capi.topk(bufs[b].data_ptr(), vals.data_ptr(), idx.data_ptr(), dt, sh, -1, k, 1, 1, ptr,
                                                    wsb + 256, stream), nb),
                          timed(lambda b: capi.softmax_topk(bufs[b].data_ptr(), 0, vals.data_ptr(), idx.data_ptr(), dt, sh, -1, k, 1,
                                                            ptr, wsb + 256, stream), nb),
                          timed(lambda b: capi.topk(bufs[b].data_ptr(), vals.data_ptr(), idx.data_ptr(), dt, sh, -1, k, 0, 1, ptr,
                                                    wsb + 256, stream), nb)]
                    if args.eager:
                        continue
                    if kind == "normal":
                        base = us
                    line = {"case": name, "path": capi.measure_path(dt, sh, -1, k), "topk_us": round(us[0], 1),
                            "fused_us": round(us[1], 1), "smallest_us": round(us[2], 1)}
                    if base is not None:
                        slow = [w for w, v, bv in zip(("topk", "fused", "smallest"), us, base) if v > 3 * bv and v > 30]
                        if slow:
                            line["over_3x_normal"] = slow
                    print(json.dumps(line), flush=True)
        return

    c1 = synth.classifier_logits(1, 1000, synth.SEEDS["C1"])
    c2 = synth.classifier_logits(256, 1000, synth.SEEDS["C2"])
    c2h = c2.astype(np.float16)
    c3 = synth.llm_logits(64, 128256, synth.SEEDS["C3"])
    c4 = synth.grid_values(8, 262144, synth.SEEDS["C4"])
    c5 = synth.detection_scores(16, 80, 8400, synth.SEEDS["C5"])

    softmax_case("C1 softmax [1,1000] f32", c1, -1)
    select_case("C1 topk k=5 [1,1000] f32", c1, 5, False)
    select_case("C1 softmax+topk k=5 [1,1000] f32", c1, 5, True)
    softmax_case("C2 softmax [256,1000] f32", c2, -1)
    softmax_case("C2 softmax [256,1000] f16", c2h, -1)
    select_case("C2 topk k=5 [256,1000] f32", c2, 5, False)
    select_case("C2 softmax+topk k=5 [256,1000] f32", c2, 5, True)
    select_case("C2 softmax+topk k=5 [256,1000] f16", c2h, 5, True)
    softmax_case("C3 softmax [64,128256] f32", c3, -1)
    select_case("C3 topk k=50 [64,128256] f32", c3, 50, False)
    select_case("C3 softmax+topk k=50 [64,128256] f32", c3, 50, True)
    c3h = c3.astype(np.float16)
    select_case("C3 softmax+topk k=50 [64,128256] f16", c3h, 50, True)
    select_case("C3 topk k=50 [64,128256] f16", c3h, 50, False)
    # the same logits after a round trip through bfloat16: equal values straddle the k-th place in most rows
    c3q = np.ascontiguousarray((c3.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32))
    select_case("C3 bf16-valued softmax+topk k=50 [64,128256] f32", c3q, 50, True)
    # every row sorted: the top of a row sits in neighbouring lanes of one chunk
    select_case("C3 sorted-rows softmax+topk k=50 [64,128256] f32", np.ascontiguousarray(np.sort(c3, axis=-1)), 50, True)
    # constrained decoding: all but 20 logits of every row masked with -inf, fewer than k are left
    c3m = np.full_like(c3, -np.inf)
    c3m[:, 1000:128000:6350] = c3[:, 1000:128000:6350]
    select_case("C3 masked-rows softmax+topk k=50 [64,128256] f32", c3m, 50, True)
    # int8-like logits: 256 levels, hundreds of elements equal the value at the k-th place
    c3i = np.ascontiguousarray(np.clip(np.round(c3 * 16), -128, 127).astype(np.float32) * np.float32(0.125))
    select_case("C3 int8-valued softmax+topk k=50 [64,128256] f32", c3i, 50, True)
    select_case("C3 int8-valued topk k=50 [64,128256] f32", c3i, 50, False)
    # the sampling entry point: temperature 0.8 and the nucleus count for top_p = 0.9 in the same call
    sampling_case("C3 sampling softmax+topk k=50 [64,128256] f32, scale 1.25, top_p 0.9", c3, 50, 1.25, 0.9)
    sampling_case("C2 sampling softmax+topk k=5 [256,1000] f32, scale 1.25, top_p 0.9", c2, 5, 1.25, 0.9)
    sampling_case("sampling softmax+topk k=40 [64,8192] f32, scale 1.25, top_p 0.9", np.ascontiguousarray(c3[:, :8192]), 40, 1.25, 0.9)
    softmax_case("C4 softmax [8,262144] f32", c4, -1)
    select_case("C4 topk k=1024 [8,262144] f32 (ties)", c4, 1024, False)
    select_case("C4 softmax+topk k=1024 [8,262144] f32", c4, 1024, True)
    select_case("C4 topk smallest k=1024 [8,262144] f32, sorted", c4, 1024, False, largest=0, sorted_=1)
    select_case("C4 topk smallest k=1024 [8,262144] f32, sorted = 0", c4, 1024, False, largest=0, sorted_=0)
    softmax_case("C5 softmax axis 1 [16,80,8400] f32", c5, 1)
    if args.only in "C5 chain softmax axis 1 -> max -> topk k=300":
        # the detection-style chain: softmax over classes, per-anchor class maximum, top-k anchors
        bufs = buffers(c5)
        p = torch.empty_like(bufs[0])
        m = torch.empty((16, 8400), dtype=torch.float32, device="cuda")
        vals = torch.empty((16, 300), dtype=torch.float32, device="cuda")
        idx = torch.empty((16, 300), dtype=torch.int32, device="cuda")
        nb = max(capi.softmax_workspace_bytes(F32, c5.shape, 1), capi.topk_workspace_bytes(F32, (16, 8400), -1, 300))
        ws, ptr = workspace(nb + 256)

        def chain(b):
            capi.softmax(bufs[b].data_ptr(), p.data_ptr(), F32, c5.shape, 1, 0, 0.0, ptr, nb + 256, stream)
            capi.reduce_max(p.data_ptr(), m.data_ptr(), F32, c5.shape, 1, stream)
            capi.topk(m.data_ptr(), vals.data_ptr(), idx.data_ptr(), F32, (16, 8400), -1, 300, 1, 1, ptr, nb + 256, stream)
        report("C5 chain softmax axis 1 -> max -> topk k=300", timed(chain, len(bufs)), c5.nbytes + 16 * 300 * 8)

        def chain_one_pass(b):   # softmax and class maximum in one read, then the same top-k
            capi.softmax_reduce_max(bufs[b].data_ptr(), m.data_ptr(), F32, c5.shape, 1, ptr, nb + 256, stream)
            capi.topk(m.data_ptr(), vals.data_ptr(), idx.data_ptr(), F32, (16, 8400), -1, 300, 1, 1, ptr, nb + 256, stream)
        report("C5 chain (softmax+max in one pass) -> topk k=300", timed(chain_one_pass, len(bufs)), c5.nbytes + 16 * 300 * 8)

    def nms_case(name, boxes, scores, per_class, iou_thr, score_thr):
        if args.only not in name:
            return
        B, C, N = scores.shape
        bx, sc = torch.from_numpy(boxes).cuda(), torch.from_numpy(scores).cuda()
        cap = B * C * (min(N, per_class) if per_class > 0 else min(N, 2048))
        out = torch.empty((cap, 3), dtype=torch.int32, device="cuda")
        count = torch.zeros(2, dtype=torch.int32, device="cuda")
        nb = capi.nms_workspace_bytes(B, C, N, per_class)
        ws, ptr = workspace(nb + 256)
        us = timed(lambda b: capi.nms(bx.data_ptr(), sc.data_ptr(), out.data_ptr(), cap, count.data_ptr(), F32, B, C, N, 0,
                                      per_class, iou_thr, score_thr, ptr, nb + 256, stream), 1)
        m = int(count.cpu()[0])
        if us is None:
            print(json.dumps({"case": name, "eager": True, "selected": m}), flush=True)
            return
        print(json.dumps({"case": name, "us_per_call": round(us, 2), "selected": m,
                          "algorithmic_bytes": boxes.nbytes + scores.nbytes + 12 * m,
                          "algorithmic_GBps": round((boxes.nbytes + scores.nbytes + 12 * m) / us / 1e3, 1)}), flush=True)

    # detection head after the chain above: softmax scores [16,80,8400], uniform boxes, the usual thresholds
    rng = np.random.default_rng(synth.SEEDS["C5"] + 1)
    ctr, size = rng.random((16, 8400, 2), dtype=np.float32), rng.random((16, 8400, 2), dtype=np.float32) * np.float32(0.2)
    boxes = np.ascontiguousarray(np.concatenate([ctr - size / 2, ctr + size / 2], axis=-1))
    e = np.exp(c5 - c5.max(axis=1, keepdims=True))
    nms_case("C5 nms [16,80,8400] f32 iou 0.45 score 0.25 max 100", boxes, np.ascontiguousarray((e / e.sum(axis=1, keepdims=True))
             .astype(np.float32)), 100, 0.45, 0.25)
    nms_case("nms one image [1,80,8400] f32 iou 0.45 score 0.25 max 100", boxes[:1], np.ascontiguousarray((e / e.sum(axis=1, keepdims=True))
             .astype(np.float32)[:1]), 100, 0.45, 0.25)
    # the longest walk one (batch, class) pair can ask for: 2048 candidates, none suppressed early
    nms_case("nms [1,1,2048] f32 all candidates, iou 0.7", boxes[:1, :2048], rng.random((1, 1, 2048), dtype=np.float32), 0,
             0.7, 0.0)
    nms_case("nms [8,80,2048] f32 all candidates, iou 0.5 max 200", boxes[:8, :2048],
             rng.random((8, 80, 2048), dtype=np.float32), 200, 0.5, 0.0)
    capi.event_destroy(e0)
    capi.event_destroy(e1)
    capi.stream_destroy(stream)


if __name__ == "__main__":
    main()
