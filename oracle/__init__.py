"""CPU oracle for the quantized (Sage-style) attention path.  TEST INFRASTRUCTURE ONLY.

Nothing here is product code: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package, and only as the checker.
The product path (``ksanadit_amd``) never imports it and has no CPU fallback.

Functions and what pins each of them:

* ``sdpa_ref.sdpa_ref``           restates ksana/operations/attention/backends/sdpa.py:47-79
  (three transposes around ``F.scaled_dot_product_attention``).  Pinned by a float64
  brute-force ``softmax(QK^T * scale) V`` on small shapes (tests/test_oracle.py).
* ``quant_ref.k_mean_ref``        per-(b,h,d) mean of K over the sequence, the ``km`` of
  ksana/operations/attention/backends/sage_sla.py:198, with the summation order frozen so a
  GPU kernel can reproduce it bit for bit.  Pinned by a pure-Python scalar replay of the
  order, by agreement with a float64 mean to fp32 rounding error, and by the closed form
  for constant columns.
* ``quant_ref.quant_q_ref`` / ``quant_k_ref``   per-block INT8 with fp32 scales
  (stage order and block sizes (128, 64) from sage_sla.py:202-204).  Pinned by a scalar
  pure-Python second implementation, hand-computed blocks (ties, single outlier, all-equal,
  all-zero, ragged tail) and the invariants |x - scale*x_i8| <= scale/2, max|x_i8| == 127.
* ``quant_ref.quant_v_ref``       per-channel FP8 e4m3fn V (sage_sla.py:222-228).  Pinned by
  an exhaustive 256-entry decode table built from the format definition, round-trip
  exactness, saturation at +-448 and the scalar second implementation.
  With ``smooth_v`` the channel mean (the K-mean function, pinned above) is taken off first and returned;
  pinned by recomputing the codes from the centred values with the plain rule, by the dequantisation bound on
  the deviation, and by the attention identity ``P (V - m) + m == P V`` (a per-channel offset of V moves the
  emulated output by that offset, tests/test_oracle.py).
* ``sage_emul_ref.sage_emul_ref`` dequantised emulation of the fused kernel.  Pinned by its
  distance to ``sdpa_ref`` (it is an approximation by construction) and by the exact
  invariants: V == 1 -> O == 1, key-permutation equivariance, K-offset invariance.
* ``k_lens`` / ``block_mask`` arguments of ``sdpa_ref`` and ``sage_emul_from_quant``: the per-batch key
  count of ksana/operations/attention/backends/flash_attn.py:131-139 and the 128 x 64 block mask of
  backends/radial_sage_attn/radial_sage_attn.py:150-176.  Pinned by an independent formulation each
  (attention on the cut / gathered operands, float64 brute force), tests/test_oracle.py.
* ``prep_ref``                    RMSNorm over the token row (ksana/operations/ops.py:62-72) and the 3-axis
  rotary embedding (ksana/utils/rope.py:61-128, ksana/models/wan/wan_model.py:51-58,677-684).  Pinned by
  ``torch.nn.functional.rms_norm`` (the routine the reference's default configuration dispatches to),
  float64 brute force, an independent real-arithmetic form of the rotation and the rotation's
  invariants (tests/test_prep_oracle.py).  The summation order behind ``mean(x^2)`` is frozen by this
  repository (not stated by the reference); against the library routine it moves about one bf16 result in
  10^5 by one ulp.

The arithmetic the reference runs lives in the third-party package ``sageattention``
(call site ksana/operations/attention/backends/sage_attn.py:75-81), which is neither
vendored nor version-pinned in the reference and is not installed here.  The exact bits
that package would produce for q_int8/k_int8/q_scale/k_scale are therefore
**parity unpinned**; the quantizer specification below is this repository's own, and the
attention output is anchored on the reference's torch SDPA backend within a stated tolerance.
"""
