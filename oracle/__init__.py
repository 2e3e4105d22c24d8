"""CPU oracle for the MoE-layer hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU, the algorithm of the reference's MoE layer
(router top-k + softmax, expert histogram / offsets / routing metadata, grouped
up-/down-projection with SwiGLU, weighted combine, and the full backward).  It is
the checker the HIP path is compared against; nothing in the product package may
import it.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
use it.

Pinning status (what independent fact each function is checked against lives in
tests/test_oracle_*.py):

  routing.topk_softmax            pinned: brute force with engineered ties; torch.topk on tie-free rows;
                                  closed-form softmax
  routing.count_cumsum            pinned: numpy.bincount / cumsum, sum / monotonic invariants
  routing.tc_topk_router_metadata pinned: permutation / stability / inverse invariants
  routing.general_routing_router_metadata   pinned: same invariants + brute-force loops
  routing.token_choice_rounding   pinned: invariants (multiples of the tile, |delta| <= tile/2, TC picks
                                  precede non-picks) + brute force on tiny inputs
  moe_math.moe_torch_backend      pinned: reduces to F.linear / F.silu / index_add; E=1 dense MLP special case
  moe_math.* explicit backward    pinned: torch.autograd through the restated forward in fp64
  moe_math.switch_aux_loss        pinned: closed form (uniform routing -> 1)
  moe_math.activation_forward / activation_backward   pinned: torch.nn.functional routines; autograd in fp64
  moe_math bias terms (db1, db2, ds bias term)        pinned: torch.autograd through the restated forward in fp64
  fp8.*                           PARITY UNPINNED against the reference, which has no fp8 implementation, test or
                                  number; the format itself is pinned: decode table and element rounding against
                                  torch.float8_e4m3fn, block scales against their defining inequalities
"""
