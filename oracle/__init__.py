"""CPU oracle for the Megalodon fused-op hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``megalodon_amd/`` imports this
package; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` do, and only as the checker.  Each function restates the
reference algorithm in float64 (NumPy / PyTorch-CPU) and cites the reference
lines it follows.

Pinning status (what independently fixes each function; see tests/test_oracle_*.py):

* ``cema.calc_coeffs``, ``cema.ema_weight_fwd``, ``cema.ema_weight_bwd``:
  pinned by closed forms (geometric series for N=1, k[0], 2*pi phase
  invariance), torch autograd over the complex128 closed form, central finite
  differences, and -- where ``oracle/_ref`` is built -- the reference's own
  C++ CPU path compiled from /root/reference.
* ``cema.ema_bias_fwd/bwd``, ``cema.ema_hidden_fwd/bwd`` (carried state):
  pinned by the EMA recurrence h_t = q h_(t-1) + p x_t run step by step,
  by splitting a sequence in two with the state handed over, by autograd over
  the complex128 closed forms and by the reference's EMAParametersCPU* /
  EMAHiddenCPU* operators (``oracle/_ref``).
* ``fftconv.fftconv_fwd/bwd``: pinned by brute-force O(L^2) causal sums,
  ``numpy.convolve``, the EMA recurrence (no FFT involved) and autograd.
* ``timestep_norm.group_timestep_norm_fwd/bwd``: pinned by brute-force
  per-prefix statistics, autograd over the cumulative-sum closed form, finite
  differences and ``oracle/_ref`` (reference C++ CPU path) where built.
* ``attention.chunk_attention_fwd/bwd``: pinned by row-0 / permutation /
  softmax-normalisation properties and autograd over the textbook formula
  (which is the reference's own unfused branch).
* ``philox.philox4x32_10`` and the masks built on it (DropKey, dropout):
  pinned by the known-answer vectors Random123 ships for Philox4x32-10 and by
  element-by-element evaluation.  The reference's masks come from curand's
  per-thread streams and are NOT reproduced: parity unpinned for the mask
  stream itself; what is checked is the operator under an identical mask.

The reference ships no tests, golden vectors or fixtures for any of these
functions, so none of them can be checked against reference-held vectors.
"""
