"""The library's launches recorded into a HIP graph (callers such as the bench replay them; the launchers clear
their accumulators with fill kernels, never with memset nodes): every replay must return what the same calls
return eagerly on the inputs the buffers hold at that moment.  The graph is replayed several times with new
inputs and eager work and synchronisations in between, and every replay is compared bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402


def test_replays_equal_eager_results():
    dev = torch.device("cuda")
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    N, K, E, Tk, top_k, D = 512, 1024, 4, 96, 2, 256
    w = torch.empty(K, N, device=dev).normal_(0, 0.02, generator=gen)
    q8, s8 = T.quantize_int8(w, per_channel=True)
    fw8 = T.FrozenWeight(q8.reshape(-1), T.W_INT8, s8, N, K, N)
    p4, s4 = T.quantize_int4_per_group(w.reshape(N, K), 128)
    fw4 = T.FrozenWeight(p4, T.W_INT4_GROUP, s4, N, K, 1, 128)
    # K = 4096: the row-block decode kernel runs int8 in two reduction slices whose sums meet in the workspace
    # (16 rows, 24 rows in two tiles, fp32 compute)
    wk = torch.empty(4096, N, device=dev).normal_(0, 0.02, generator=gen)
    q8k, s8k = T.quantize_int8(wk, per_channel=True)
    fw8k = T.FrozenWeight(q8k.reshape(-1), T.W_INT8, s8k, N, 4096, N)
    experts = []
    for _ in range(E):
        we = torch.empty(D, D, device=dev).normal_(0, 0.02, generator=gen)
        qe, se = T.quantize_int8(we, per_channel=True)
        experts.append(T.FrozenWeight(qe.reshape(-1), T.W_INT8, se, D, D, D))
    gw = T.GroupedFrozenWeights(experts)

    # static inputs, refilled before every replay
    wsrc = torch.empty(K, N, device=dev)
    x1, x16, x64 = (torch.empty(m, K, device=dev, dtype=torch.bfloat16) for m in (1, 16, 64))
    dy64 = torch.empty(64, N, device=dev, dtype=torch.bfloat16)
    xf = torch.empty(16, K, device=dev)
    x16k, x24k = (torch.empty(m, 4096, device=dev, dtype=torch.bfloat16) for m in (16, 24))
    xfk = torch.empty(5, 4096, device=dev)
    tok = torch.empty(Tk, D, device=dev, dtype=torch.bfloat16)
    idx = torch.empty(Tk, top_k, device=dev, dtype=torch.int32)
    wts = torch.empty(Tk, top_k, device=dev, dtype=torch.bfloat16)
    rows = Tk * top_k
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)

    def refill(seed):
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        wsrc.normal_(0, 0.02, generator=g)
        for t in (x1, x16, x64, tok, x16k, x24k):
            t.copy_(torch.empty(t.shape, device=dev).normal_(0, 1, generator=g))
        dy64.copy_(torch.empty(64, N, device=dev).normal_(0, 1e-2, generator=g))
        xf.normal_(0, 1, generator=g)
        xfk.normal_(0, 1, generator=g)
        idx.copy_(torch.randint(0, E, (Tk, top_k), device=dev, generator=g).to(torch.int32))
        wts.copy_(torch.softmax(torch.empty(Tk, top_k, device=dev).normal_(0, 1, generator=g), dim=1))

    def work():
        out = {}
        out["q8"], out["s8"] = T.quantize_int8(wsrc, per_channel=True)          # column maxima through atomics
        out["qt"], out["st"] = T.quantize_int8(wsrc, per_channel=False)
        out["p4"], out["s4"] = T.quantize_int4_per_group(wsrc, 128)
        out["y1_4"] = T.qlinear_forward(x1, fw4, T.BF16, workspace=ws)
        out["y1_8"] = T.qlinear_forward(x1, fw8, T.BF16, workspace=ws)
        out["y16"] = T.qlinear_forward(x16, fw8, T.BF16, workspace=ws)
        out["y64"] = T.qlinear_forward(x64, fw4, T.BF16, workspace=ws)
        out["dx64"] = T.qlinear_backward_input(dy64, fw8, T.BF16, workspace=ws)
        out["yf"] = T.qlinear_forward(xf, fw8, T.F32, workspace=ws)
        out["y16k"] = T.qlinear_forward(x16k, fw8k, T.BF16, workspace=ws)
        out["y24k"] = T.qlinear_forward(x24k, fw8k, T.BF16, workspace=ws)
        out["yfk"] = T.qlinear_forward(xfk, fw8k, T.F32, workspace=ws)
        dmap, offs = T.moe_build_dispatch_map(idx, E)                            # counters, scans
        packed = T.moe_dispatch(tok, idx, dmap, offs, rows, out=torch.empty(rows, D, device=dev, dtype=torch.bfloat16))
        ye = T.qlinear_grouped_forward(packed, offs, gw, T.BF16, T.BF16, workspace=ws,
                                       out=torch.empty(rows, D, device=dev, dtype=torch.bfloat16))
        out["dmap"], out["offs"], out["packed"], out["ye"] = dmap, offs, packed, ye
        out["comb"] = T.moe_combine(ye, idx, wts, dmap, offs)
        return out

    refill(100)
    work()                                                           # warm up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = work()
    torch.cuda.synchronize()

    for rep in range(4):
        refill(200 + rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = {k: v.clone() for k, v in captured.items()}
        want = work()                                                # the program's own eager work between replays
        torch.cuda.synchronize()
        for k in want:
            assert torch.equal(got[k], want[k]), (rep, k)
    assert not np.isnan(got["comb"].float().cpu().numpy()).any()


def test_replays_of_the_large_forward_kernels_and_the_few_row_gradient():
    # the int4 and int8 forward kernels that keep the weight out of the shared operand tiles (first launched inside
    # the capture: they raise their LDS limit there), the grouped int8 form, and the few-row input gradient with its
    # gradient piece staged through LDS (three residue classes) and its adding pass
    dev = torch.device("cuda")
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)

    def int8(n, k):
        q, s = T.quantize_int8(torch.empty(k, n, device=dev).normal_(0, 0.02, generator=gen), per_channel=True)
        return T.FrozenWeight(q.reshape(-1), T.W_INT8, s, n, k, n)

    N, K, M = 2048, 640, 4096
    fw8 = int8(N, K)
    p4, s4 = T.quantize_int4_per_group(torch.empty(N, 512, device=dev).normal_(0, 0.02, generator=gen), 128)
    fw4 = T.FrozenWeight(p4, T.W_INT4_GROUP, s4, N, 512, 1, 128)
    E, rows = 8, 16384
    gw = T.GroupedFrozenWeights([int8(512, 256) for _ in range(E)])
    offsets = torch.tensor([0, 2000, 2000, 4100, 6148, 9000, 12000, 15000, rows], dtype=torch.int32, device=dev)
    fwd = int8(1536, 1024)                                           # K mod N = 1024: three residue classes of rows
    x8 = torch.empty(M, K, device=dev, dtype=torch.bfloat16)
    x4 = torch.empty(M, 512, device=dev, dtype=torch.bfloat16)
    xg = torch.empty(rows, 256, device=dev, dtype=torch.bfloat16)
    dy = torch.empty(16, 1536, device=dev, dtype=torch.bfloat16)
    ws = torch.empty(1 << 22, dtype=torch.uint8, device=dev)

    def refill():
        for t, std in ((x8, 1.0), (x4, 1.0), (xg, 1.0), (dy, 1e-2)):
            t.copy_(torch.empty(t.shape, device=dev).normal_(0, std, generator=gen))

    def run():
        return (T.qlinear_forward(x8, fw8, T.BF16, T.BF16), T.qlinear_forward(x4, fw4, T.BF16, T.F32),
                T.qlinear_grouped_forward(xg, offsets, gw, T.BF16, T.BF16),
                T.qlinear_backward_input(dy, fwd, T.BF16, T.F32, workspace=ws))

    refill()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            outs = run()
    torch.cuda.synchronize()
    for rep in range(3):
        refill()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = run()
        torch.cuda.synchronize()
        for got, ref in zip(outs, want):
            assert torch.equal(got, ref), rep
