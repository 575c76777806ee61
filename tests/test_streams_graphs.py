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
