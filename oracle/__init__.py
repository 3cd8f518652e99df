"""CPU oracle for the GEMM / quantisation hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module: it is the checker used by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``.  Every function restates, in plain
numpy / CPU torch, what the reference computes and cites the reference
file:line it follows.

Parity status (what pins each function is listed next to it):

* ``gemm.ref_gemm*``            pinned  (closed form: fp32 ``torch.matmul``, the reference's own oracle)
* ``mxfp4.mxfp4_to_f32``        pinned  (OCP-MX e2m1 table, reference LUT)
* ``mxfp4.e8m0_to_f32``         pinned  (2**(b-127) closed form + the two special bytes)
* ``mxfp4.mxfp4_quant``         pinned  (outputs of the reference's own kernel under Triton's CPU interpreter,
                                committed as tests/golden/mxfp4_quant_vectors.npz; hand-derived known
                                answers; brute force vs. nearest-value search)
* ``mxfp4.hadamard32``          pinned  (Sylvester matrix from scipy, H*H = 32 I, norm preservation)
* ``schedule.*``                pinned  (brute-force bijection / exact-cover checks)
* ``selector.estimate_lds_bytes`` pinned (reference known-answer tests)
* ``selector.compute_sk_grid``  pinned  (hand-checked cases)
* tile *choice* of the analytical model: parity unpinned (the reference delegates it to an
  external C++ library that is not part of the reference tree; it never affects numerics).
"""
