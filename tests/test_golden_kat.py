"""Known-answer vectors worked out by hand from the reference's definitions (tests/golden/README.md): the oracle on
the CPU, the HIP kernels on the GPU."""

import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import moe_math as M
from oracle import routing as R

KAT = json.loads((Path(__file__).parent / "golden" / "routing_kat.json").read_text())
META_KEYS = ["expert_frequency", "expert_frequency_offset", "s_scatter_idx", "x_gather_idx", "s_reverse_scatter_idx",
             "num_activated_expert_per_token_offset"]


def test_oracle_topk_softmax():
    k = KAT["topk_softmax"]
    s, i = R.topk_softmax(np.asarray(k["logits"], dtype=np.float32), k["K"])
    assert i.tolist() == k["indices"]
    np.testing.assert_allclose(s, np.asarray(k["scores"]), rtol=1e-6)


def test_oracle_metadata():
    k = KAT["tc_metadata"]
    got = R.tc_topk_router_metadata(np.asarray(k["indices"], dtype=np.int32), k["E"])
    for key in META_KEYS:
        assert got[key].tolist() == k[key], key
    cnt, cum = R.count_cumsum(np.asarray(k["indices"], dtype=np.int32).reshape(-1), k["E"])
    assert cnt.tolist() == k["expert_frequency"] and cum.tolist() == k["expert_frequency_offset"][1:]
    g = KAT["general_metadata"]
    got = R.general_routing_router_metadata(np.asarray(g["token_idx"], dtype=np.int32),
                                            np.asarray(g["expert_idx"], dtype=np.int32), g["T"], g["E"])
    for key in META_KEYS:
        assert got[key].tolist() == g[key], key


def test_oracle_softmax_topk_bwd_rounding_swiglu():
    k = KAT["softmax_topk_bwd"]
    d = M.softmax_topk_bwd(torch.tensor(k["dscores"]), torch.tensor(k["scores"]), torch.tensor(k["indices"]), k["E"])
    np.testing.assert_allclose(d.numpy(), np.asarray(k["dlogits"]), atol=1e-7)
    r = KAT["rounding"]
    for mode in ("nr", "up", "down"):
        assert R.round_half_even_multiple(np.asarray(r["freq"], dtype=np.int32), r["tile"], mode).tolist() == r[mode]
    s = KAT["swiglu"]
    np.testing.assert_allclose(M.swiglu(torch.tensor(s["z"], dtype=torch.float64)).numpy(), np.asarray(s["y"]), rtol=1e-12)
    np.testing.assert_allclose(M.activation_forward(torch.tensor(s["z"], dtype=torch.float64), "swiglu").numpy(),
                               np.asarray(s["y"]), rtol=1e-12)


@pytest.mark.gpu
def test_hip_kernels_on_known_answers(dev):
    from sonicmoe.functional import TC_topk_router_metadata, backward, forward, general_routing_router_metadata

    k = KAT["topk_softmax"]
    for dtype in (torch.float32, torch.bfloat16):  # 0.1 and 0.7 round in bf16 but keep their order and their tie
        logits = torch.tensor(k["logits"], dtype=dtype, device=dev)
        T = logits.size(0)
        s = torch.empty(T, k["K"], dtype=torch.float32, device=dev)
        i = torch.empty(T, k["K"], dtype=torch.int32, device=dev)
        forward._topk_fwd(logits, k["K"], s, i, True)
        assert i.cpu().tolist() == k["indices"]
        np.testing.assert_allclose(s.cpu().numpy(), np.asarray(k["scores"]), rtol=1e-5)

    m = KAT["tc_metadata"]
    idx = torch.tensor(m["indices"], dtype=torch.int32, device=dev)
    got = TC_topk_router_metadata(idx, torch.empty(m["E"], dtype=torch.int32, device=dev), m["K"])
    names = ["expert_frequency_offset", "x_gather_idx", "s_scatter_idx", "s_reverse_scatter_idx",
             "num_activated_expert_per_token_offset"]
    for key, t in zip(names, got):
        assert t.cpu().tolist() == m[key], key
    from sonicmoe import count_cumsum

    cnt, cum = count_cumsum(idx.view(-1), m["E"], do_cumsum=True)
    assert cnt.cpu().tolist() == m["expert_frequency"] and cum.cpu().tolist() == m["expert_frequency_offset"][1:]

    g = KAT["general_metadata"]
    got = general_routing_router_metadata(torch.zeros(6, device=dev), torch.tensor(g["token_idx"], dtype=torch.int32, device=dev),
                                          torch.tensor(g["expert_idx"], dtype=torch.int32, device=dev), g["T"], g["E"])
    for key, t in zip(["expert_frequency"] + names, got):
        assert t.cpu().tolist() == g[key], key

    b = KAT["softmax_topk_bwd"]
    dl = torch.zeros(1, b["E"], dtype=torch.float32, device=dev)
    backward._softmax_topk_bwd(dl, None, torch.tensor(b["dscores"], device=dev), torch.tensor(b["scores"], device=dev),
                               torch.tensor(b["indices"], dtype=torch.int32, device=dev), 2)
    np.testing.assert_allclose(dl.cpu().numpy(), np.asarray(b["dlogits"]), atol=1e-7)
