"""CPU oracle for the sparse-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it,
and only as the checker.  Every function restates, in NumPy, one function of the
reference's pure-MLX fallback and cites the reference file:line it follows.

Pinning status (what fixes each function besides its own formula):

* ``fp8.e4m3_decode``            -- closed-form bit spec; pinned against the
  reference's edge-byte known answers and against torch's independent
  ``float8_e4m3fn`` decoder for all 254 non-NaN bytes.
* ``fp8.e8m0_decode``            -- pinned against the reference-held table
  rule (byte 0 or 255 -> 0, else 2**(b-127)).
* ``fp8.e4m3_encode``, ``fp8.quantize_*`` -- producer side.  The reference
  delegates to MLX ``mx.to_fp8`` / ``mx.quantize`` whose source is not in the
  tree; ``quantize_per_tensor`` and ``quantize_mxfp8`` are pinned by the two
  seeded receipts the reference holds (bench/tilelang_ports/sparse_mla_fp8.json
  ``parity.fp8_vs_bf16`` and sparse_mla_blockscaled.json
  ``parity.blockscaled_vs_bf16``, regenerated in
  tests/test_oracle_reference_receipts.py), ``quantize_per_token`` by the
  reference's own producer kernel text, ``e4m3_encode`` by round-trip exactness
  on the e4m3 grid and nearest-value brute force.  Left open by the receipts:
  the rounding of an MXFP8 exponent exactly half-way between two integers
  (cannot occur for a float amax) and ties of ``mx.to_fp8`` on exact code
  midpoints (assumed to-even, as every IEEE-style converter).
* ``topk.topk_selector_oracle``  -- pinned by the reference tests' exact-order
  known answers, sentinel cases and an O(T^2) brute-force ranker.
* ``sparse_mla.sparse_mla_oracle`` -- pinned against a per-token loop
  formulation, ``torch.softmax`` / ``torch.logsumexp`` closed forms and the
  invariants the reference tests pin (all-invalid row -> zeros, duplicated
  index = doubled weight, permutation invariance).
* ``indexer.indexer_scores_oracle`` / ``indexer_topk_oracle`` -- pinned against an
  explicit four-loop evaluation, the head-sum-first identity, ``np.argpartition``'s
  set on distinct scores and the reference's rope known answers.
* ``vecmat.*``                   -- pinned against float64 ``W_deq @ x`` with
  torch's independent e4m3 decoder.
* ``mla_absorb.*``               -- pinned by the reference's identity absorbed == standard
  decode and by explicit einsum loops.
* ``sparse_mla.sparse_mla_bwd_oracle`` -- pinned by central finite differences of the forward
  oracle in float64 and by torch autograd through a dense softmax attention restricted to the
  selected keys.
* ``dsa_loss.*``                 -- pinned by closed forms (zero rows and a uniform index give
  log(Sk) - log(sq + 1); an index equal to the log of the attention distribution on a full
  row gives 0) and an explicit triple loop with a sparse mask.
"""
