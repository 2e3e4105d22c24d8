"""smoe_routing_metadata_static (the entry point that allocates nothing: its scratch tables are a device array inside
the library) against smoe_routing_metadata (caller-supplied workspace), through the C ABI, bit for bit, on two calls
in a row of which the second is smaller, so that whatever the first call left in the shared array is in the way."""

import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_both(lib, dev, expert_idx, token_idx, T, E, K):
    TK = expert_idx.numel()
    i32 = dict(dtype=torch.int32, device=dev)

    def outputs():
        # garbage, not zeros: every element has to be written by the call
        return [torch.full((n,), -7, **i32) for n in (E, E + 1, TK, TK, TK, T + 1)]

    ws_bytes = lib.smoe_routing_metadata_workspace_bytes(TK, E)
    ws = torch.full((max(ws_bytes, 4),), 0x5A, dtype=torch.uint8, device=dev)
    ref = outputs()
    tok_ptr = None if token_idx is None else token_idx.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.smoe_routing_metadata(expert_idx.data_ptr(), tok_ptr, TK, T, E, K, *[t.data_ptr() for t in ref],
                                   ws.data_ptr(), ws_bytes, stream)
    assert rc == 0, lib.smoe_last_error()
    got = outputs()
    rc = lib.smoe_routing_metadata_static(expert_idx.data_ptr(), tok_ptr, TK, T, E, K, *[t.data_ptr() for t in got],
                                          stream)
    assert rc == 0, lib.smoe_last_error()
    torch.cuda.synchronize()
    for name, a, b in zip(["freq", "off", "gidx", "sidx", "ridx", "tok_off"], got, ref):
        assert torch.equal(a, b), name
    return got


def test_static_scratch_entry_matches_workspace_entry(dev):
    from oracle import routing as R
    from sonicmoe import _lib

    lib = _lib.lib()
    assert lib.smoe_routing_metadata_static_capacity() == 4 << 20
    rng = np.random.default_rng(5)
    # first call: many segments and experts; second call: smaller in both, so stale table entries of the first lie
    # beyond and between the entries the second one uses
    for T, E, K in [(16384, 128, 8), (1000, 24, 3)]:
        idx = np.stack([rng.choice(E, size=K, replace=False) for _ in range(T)]).astype(np.int32)
        got = _call_both(lib, dev, torch.from_numpy(idx.reshape(-1)).to(dev), None, T, E, K)
        meta = R.tc_topk_router_metadata(idx, E)
        assert np.array_equal(got[0].cpu().numpy(), meta["expert_frequency"])
        assert np.array_equal(got[3].cpu().numpy(), meta["s_scatter_idx"])
    # general routing (token_idx given), smaller again
    T, E = 300, 16
    keep = rng.random((T, E)) < 0.2
    tok, exp = np.nonzero(keep)
    _call_both(lib, dev, torch.from_numpy(exp.astype(np.int32)).to(dev), torch.from_numpy(tok.astype(np.int32)).to(dev),
               T, E, 1)


def test_static_scratch_entry_rejects_sizes_beyond_its_array(dev):
    from sonicmoe import _lib

    lib = _lib.lib()
    TK, E = 1 << 22, 4096  # 2 * 4096 * 4096 * 4 bytes = 128 MiB of tables
    assert lib.smoe_routing_metadata_workspace_bytes(TK, E) > lib.smoe_routing_metadata_static_capacity()
    buf = torch.zeros(16, dtype=torch.int32, device=dev)
    p = buf.data_ptr()
    rc = lib.smoe_routing_metadata_static(p, None, TK, TK // 8, E, 8, p, p, p, p, p, None, None)
    assert rc == 4
    assert b"built-in array" in lib.smoe_last_error()
