"""yahkv_decode_attend_static (the decode attention that takes no workspace and allocates nothing) against
yahkv_decode_attend on the same inputs, through the C ABI: two calls in a row on one GPU, the second on a smaller batch,
so that the second finds the first call's partials in the library's scratch array; then a batch that does not fit."""
import numpy as np
import pytest

from helpers import rel_err, to_bf16_f32
from test_gpu_decode import setup

pytestmark = pytest.mark.gpu
TOL = 2e-3


def test_static_scratch_decode_matches_the_workspace_form_twice_in_a_row(yahkv, torch_gpu):
    torch = torch_gpu
    n_q, n_kv, hd, pt = 24, 4, 256, 64
    big = [3000, 64, 1, 777, 0, 2049, 130, 1500, 65, 4000, 31, 900]
    g, table, host, dev, rng = setup(yahkv, torch, 8, n_q, n_kv, hd, pt, big, seed=701, fill=0x7F)
    t_table = torch.from_numpy(table).cuda()
    scale = 1.0 / 16
    q = torch.from_numpy(to_bf16_f32(rng.standard_normal((len(big), n_q, hd)))).cuda().to(torch.bfloat16)
    gate = torch.from_numpy(rng.standard_normal((len(big), n_q, hd)).astype(np.float32)).cuda()
    assert yahkv.lib.yahkv_decode_static_scratch_bytes() == 32 << 20
    # outputs and inputs exist before the calls; the calls themselves must leave the device's free memory alone
    cases = [(slice(0, len(big)), gate), (slice(2, 7), None)]
    lens = [torch.tensor(big[c], dtype=torch.int32, device="cuda") for c, _ in cases]
    outs = [torch.full((len(big[c]), n_q, hd), float("nan"), device="cuda") for c, _ in cases]
    want = [yahkv.decode_attend(dev, t_table[c].contiguous(), lens[i], max(big), q[c].contiguous(), scale,
                                gate=None if gt is None else gt[c].contiguous()) for i, (c, gt) in enumerate(cases)]
    tabs = [t_table[c].contiguous() for c, _ in cases]
    qs = [q[c].contiguous() for c, _ in cases]
    gates = [None if gt is None else gt[c].contiguous() for c, gt in cases]
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for i in range(2):
        yahkv.decode_attend_static(dev, tabs[i], lens[i], max(big), qs[i], scale, outs[i], gate=gates[i])
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    for i, (c, _) in enumerate(cases):
        got, ref = outs[i].cpu().numpy(), want[i].cpu().numpy()
        assert np.all(np.isfinite(got))
        assert rel_err(got, ref) < TOL, i
        for s, n in enumerate(big[c]):
            if n == 0:
                assert not got[s].any()


def test_static_scratch_decode_refuses_what_does_not_fit(yahkv, torch_gpu):
    torch = torch_gpu
    n_seqs = 200                                       # 24 / 4 heads of 256 dims: the partials need more than 32 MiB
    g = yahkv.geometry(8, 24, 4, 256, 64, 8)
    assert yahkv.decode_workspace_bytes(g, n_seqs, 64) > yahkv.lib.yahkv_decode_static_scratch_bytes()
    dev = yahkv.DevicePools(g)
    table = torch.zeros((n_seqs, 1), dtype=torch.int32, device="cuda")
    lens = torch.ones(n_seqs, dtype=torch.int32, device="cuda")
    q = torch.zeros((n_seqs, 24, 256), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((n_seqs, 24, 256), device="cuda")
    with pytest.raises(yahkv.YahkvError) as e:
        yahkv.decode_attend_static(dev, table, lens, 64, q, 0.0625, out)
    assert e.value.status == -4
