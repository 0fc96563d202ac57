"""The entry points launch kernels on the caller's stream and nothing else (no allocation, no synchronization, no
memset), so a step can be recorded into a HIP graph. A decode step (append one token per sequence, then attention) and
a prefill chunk are captured once and replayed several times with eager work and synchronizations in between; every
replay must give what the eager call gives: bit for bit for the pools and the prefill; for the decode within 5e-4
(which wave takes which tile changes from launch to launch, and with it the running maxima the f16 numerators are
rounded against) and within 2e-3 of the oracle."""
import numpy as np
import pytest

import oracle
from helpers import rel_err, to_bf16_f32
from test_gpu_decode import setup

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("form", ["part_reduce", "one_launch", "step"])
def test_decode_step_replays_from_a_graph(yahkv, torch_gpu, form):
    torch = torch_gpu
    opt = yahkv.decode_options(one_launch=form == "one_launch", n_chunks=24, min_chunk_tiles=2)   # pairs that span several chunks
    lens = [700, 64, 1, 333]
    g, table, host, dev, rng = setup(yahkv, torch, 8, 24, 4, 256, 64, [n + 1 for n in lens], seed=21)
    t_table = torch.from_numpy(table).cuda()
    pos = torch.tensor(lens, dtype=torch.int32, device="cuda")
    seq_len = pos + 1
    q = torch.randn((4, 24, 256), device="cuda").to(torch.bfloat16)
    k = torch.randn((4, 1, 4, 256), device="cuda").to(torch.bfloat16)
    v = torch.randn((4, 1, 4, 256), device="cuda").to(torch.bfloat16)
    out = torch.empty((4, 24, 256), dtype=torch.float32, device="cuda")
    ws = torch.empty(yahkv.decode_workspace_bytes(dev.geom, 4, 701, opt), dtype=torch.uint8, device="cuda")

    def step():
        if form == "step":                            # append and attention in the step call's two dispatches
            yahkv.decode_step(dev, t_table, seq_len, 701, k[:, 0], v[:, 0], q, 0.0625, out=out, workspace=ws, opt=opt)
            return
        yahkv.append(dev, t_table, pos, k, v)
        if form == "one_launch":                      # its arrival counts start at zero: the fill kernel is captured too
            yahkv.decode_workspace_init(dev.geom, 4, 701, ws, opt)
        yahkv.decode_attend(dev, t_table, seq_len, 701, q, 0.0625, out=out, workspace=ws, opt=opt)

    step()                                            # eager: also the one-time host set-up of the library
    torch.cuda.synchronize()
    want, pools_want = out.clone(), {n: a.copy() for n, a in dev.numpy().items()}
    host_q = q.float().cpu().numpy()
    oracle.append(host, table, lens, None, k.float().cpu().numpy(), v.float().cpu().numpy())
    exact = oracle.decode_attend(host, table, [n + 1 for n in lens], host_q, 0.0625)
    assert rel_err(want.cpu().numpy(), exact) < 2e-3
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            step()
    for i in range(4):
        out.fill_(float("nan"))
        ws.random_(0, 256)                            # the workspace carries nothing from launch to launch
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert rel_err(out.cpu().numpy(), want.cpu().numpy()) < 5e-4, f"replay {i}"
        assert rel_err(out.cpu().numpy(), exact) < 2e-3, f"replay {i}"
        got = dev.numpy()
        for name, a in pools_want.items():
            assert np.array_equal(got[name], a), (name, i)
        _ = (torch.randn(1 << 20, device="cuda") * 2).sum().item()   # eager work between the replays


def test_prefill_chunk_replays_from_a_graph(yahkv, torch_gpu):
    torch = torch_gpu
    from test_gpu_prefill import build
    prefix, chunk = [200, 37], 70
    g, table, host, dev, t_table, rng, to_t = build(yahkv, torch, 8, 24, 4, 256, 64, prefix, chunk, seed=22)
    q = to_t(to_bf16_f32(rng.standard_normal((2, chunk, 24, 256))))
    t_prefix = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    out = torch.empty((2, chunk, 24, 256), dtype=torch.float32, device="cuda")
    ws = torch.empty(yahkv.prefill_workspace_bytes(dev.geom, 2, 200, chunk), dtype=torch.uint8, device="cuda")

    def step():
        yahkv.prefill_attend(dev, t_table, t_prefix, 200, q, 0.0625, out=out, workspace=ws)

    step()
    torch.cuda.synchronize()
    want = out.clone()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            step()
    for i in range(3):
        out.fill_(float("nan"))
        ws.random_(0, 256)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
        _ = (torch.randn(1 << 20, device="cuda") * 2).sum().item()
