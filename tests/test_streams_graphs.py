"""The library launches one kernel per call, asynchronously, on the stream it is handed, and allocates nothing: calls
can run on side streams (the reference splits the batch over streams, src/fmha-pipeline/fmha_forward.cu:387-419) and
inside a captured HIP graph.  Each replay is checked against the eager result, with eager work between replays."""
import numpy as np
import pytest

import oracle
from _util import TOL_FP16, max_abs, pkg, to_dev

pytestmark = pytest.mark.gpu


def test_batch_split_over_streams_matches_single_launch():
    import torch
    B, S, H, D = 4, 512, 4, 128
    q, k, v = (to_dev(x.astype(np.float16)) for x in pkg.testbed.qkv(B, S, H, D))
    whole = pkg.fmha_forward(q, k, v)
    torch.cuda.synchronize()
    parts = torch.empty_like(whole)
    streams = [torch.cuda.Stream() for _ in range(2)]           # default priority
    for i, st in enumerate(streams):
        st.wait_stream(torch.cuda.current_stream())
        sl = slice(i * B // 2, (i + 1) * B // 2)
        with torch.cuda.stream(st):
            pkg.fmha_forward(q[sl], k[sl], v[sl], o=parts[sl])  # contiguous batch slices: plain pointer offsets
    for st in streams:
        torch.cuda.current_stream().wait_stream(st)
    torch.cuda.synchronize()
    assert torch.equal(whole, parts)


def test_graph_capture_and_replay():
    import torch
    B, S, H, D = 2, 512, 4, 128
    q, k, v = (to_dev(x.astype(np.float16)) for x in pkg.testbed.qkv(B, S, H, D))
    q8 = (q.float() * 16).clamp(-448, 448).to(torch.float8_e4m3fn)
    k8 = (k.float() * 16).clamp(-448, 448).to(torch.float8_e4m3fn)
    v8 = (v.float() * 16).clamp(-448, 448).to(torch.float8_e4m3fn)
    a = to_dev(pkg.testbed.uniform((256, 256), 11).astype(np.float16))
    b = to_dev(pkg.testbed.uniform((512, 256), 12).astype(np.float16))
    o16, o8 = torch.empty_like(q), torch.empty_like(q)
    c = torch.empty((256, 512), dtype=torch.float16, device="cuda:0")

    def work():
        pkg.fmha_forward(q, k, v, o=o16)
        pkg.fmha_forward(q8, k8, v8, o=o8, q_descale=1 / 16, k_descale=1 / 16, v_descale=1 / 16)
        pkg.gemm(a, b, out=c)

    work()                                                      # eager: also does the one-time per-kernel set-up
    torch.cuda.synchronize()
    want = [t.clone() for t in (o16, o8, c)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            work()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        for t in (o16, o8, c):
            t.fill_(-1.0)                                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip((o16, o8, c), want):
            assert torch.equal(got, ref), rep
    # new inputs in the captured buffers: the replay computes on what is there now
    q.copy_(q.flip(1))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    ref = oracle.attention_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy())["O"]
    assert max_abs(o16.float().cpu().numpy(), ref) <= TOL_FP16


def test_first_calls_of_distinct_shapes_from_several_host_threads():
    # Each host thread makes the FIRST call of its own kernel instantiation in this process (head dim x precision x
    # tile), on its own stream: the one-time per-kernel set-up is thread-safe and the calls are independent.  Shapes
    # are chosen so that no other test of this module has used these instantiations before.
    import threading
    import torch
    shapes = [("f16", 1, 128, 1, 256, 32), ("f16", 1, 128, 3, 64, 192), ("f8", 1, 128, 2, 256, 64),
              ("f8", 1, 256, 2, 64, 128), ("hyb", 1, 128, 2, 64, 64), ("hyb", 1, 128, 1, 256, 96)]
    results, errors = {}, []
    inputs = {}
    for i, (mode, B, S, H, D, Skv) in enumerate(shapes):
        q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv, seed=4000 + i)
        if mode == "f16":
            dev = [to_dev(x.astype(np.float16)) for x in (q, k, v)]
            ref = oracle.attention_f32(*(x.astype(np.float16).astype(np.float32) for x in (q, k, v)))["O"]
            kw = {}
        else:
            (qc, qs), (kc, ks), (vc, vs) = (oracle.quantize_e4m3_per_tensor(x) for x in (q, k, v))
            qf, kf = oracle.e4m3_decode(qc) * qs, oracle.e4m3_decode(kc) * ks
            if mode == "f8":
                dev = [to_dev(x) for x in (qc, kc, vc)]
                ref = oracle.attention_f32(qf, kf, oracle.e4m3_decode(vc) * vs)["O"]
                kw = dict(q_descale=float(qs), k_descale=float(ks), v_descale=float(vs))
            else:
                v16 = v.astype(np.float16)
                dev = [to_dev(qc), to_dev(kc), to_dev(v16)]
                ref = oracle.attention_f32(qf, kf, v16.astype(np.float32))["O"]
                kw = dict(q_descale=float(qs), k_descale=float(ks))
        inputs[i] = (dev, kw, ref, 5e-2 if mode == "f8" else TOL_FP16)
    torch.cuda.synchronize()
    start = threading.Barrier(len(shapes))

    def worker(i):
        try:
            dev, kw, _, _ = inputs[i]
            st = torch.cuda.Stream()
            start.wait()
            with torch.cuda.stream(st):
                o = pkg.fmha_forward(*dev, **kw)
            st.synchronize()
            results[i] = o.float().cpu().numpy()
        except Exception as e:  # noqa: BLE001
            errors.append((i, e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(len(shapes)):
        _, _, ref, tol = inputs[i]
        assert max_abs(results[i], ref) <= tol, shapes[i]


def test_init_makes_a_first_call_under_capture_possible():
    # cfk_init performs every kernel's one-time set-up, so the FIRST call of a shape may sit inside a stream capture
    import torch
    assert pkg.lib().cfk_init() == 0, pkg.last_error()
    B, S, H, D = 1, 384, 5, 128                                 # 128x64 fp16 tile with an odd head count: not used above
    q, k, v = (to_dev(x.astype(np.float16)) for x in pkg.testbed.qkv(B, S, H, D, seed=77))
    o = torch.full_like(q, -1.0)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            pkg.fmha_forward(q, k, v, o=o)
    torch.cuda.current_stream().wait_stream(side)
    ref = oracle.attention_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy())["O"]
    for rep in range(2):
        o.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert max_abs(o.float().cpu().numpy(), ref) <= TOL_FP16, rep


@pytest.mark.gpu
def test_prepared_call_repeats_the_same_launch():
    # fmha_forward(..., prepare=True) fills the parameter block once; each call of the object is one cfk_fmha_forward
    import torch
    q, k, v = (to_dev(x.astype(np.float16)) for x in pkg.testbed.qkv(1, 256, 2, 64))
    ref = pkg.fmha_forward(q, k, v)
    o = torch.zeros_like(ref)
    call = pkg.fmha_forward(q, k, v, o=o, prepare=True)
    torch.cuda.synchronize()
    assert float(o.abs().max()) == 0.0          # nothing was launched yet
    for _ in range(3):
        out = call()
    torch.cuda.synchronize()
    assert out is o and torch.equal(o, ref)
