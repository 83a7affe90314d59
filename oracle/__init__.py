"""CPU oracle for the mLSTM hot path (TFLA chunkwise fwd/bwd and the recurrent decode step).

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a plain PyTorch (fp32/fp64, CPU-runnable)
restatement of the reference's *native* formulations and is only ever used as the checker by tests/,
by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``.  Nothing under
``mlstm_kernels_amd/`` imports it; the product path is the HIP library and fails loudly without it.

What pins each function (none of them is pinned by retyping its own formula):

* ``recurrent_step`` / ``recurrent_sequence``  -- closed form of one step from zero state and the
  three-way agreement recurrent == quadratic-parallel == chunkwise (tests/test_oracle.py).
* ``parallel_stablef_fw`` / ``chunkwise_fw``   -- same three-way agreement, chunk-size invariance,
  state-passing invariance, invariance under a shift of the initial stabiliser.
* ``parallel_stablef_bw`` / ``chunkwise_bw``   -- fp64 ``torch.autograd`` through an independently
  written quadratic forward whose normaliser and stabiliser are detached (that *is* the reference's
  gradient convention), plus the identity sum_d k*dK == sum_d v*dV.
* sigmoid-input-gate variants                  -- recurrent sig loop == quadratic sig == chunkwise sig,
  detached-normaliser autograd for the gradients, state passing for non-zero initial (C, n).

* ``head_normalize`` / ``head_normalize_bw``    -- torch.nn.functional.layer_norm / rms formula and fp64 autograd
  (tests/test_oracle.py).
* ``H_abs`` / ``d*_abs`` magnitude sums (``return_bounds``) are derived quantities for the test bounds, not part of
  the reference's algorithm.

The reference ships no golden vectors for this path (its tests compare live implementations).  The fixtures under
tests/golden/ are: closed-form known answers, a regression dump of this oracle, and vectors written from the
reference's OWN native functions (chunkwise forward/backward, quadratic sigmoid-gate forward/backward, decode step)
by the two make_reference_vectors*.py scripts; the oracle reproduces all of them to 1e-5.
"""
from .mlstm_ref import *  # noqa: F401,F403
