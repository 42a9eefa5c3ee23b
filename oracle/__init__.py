"""CPU oracle for the ODM-KV compression-and-decode path.

TEST INFRASTRUCTURE ONLY.  This package restates, on the CPU, the arithmetic of
the reference implementation (yiiwang118/ODM-KV) for the hot path

    score -> Lagrangian bit allocation -> Lloyd-Max quantize/pack -> decode attention

so that the HIP kernels can be compared against it.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing under ``odm-kv_amd/`` imports it, and the product raises if
its HIP library is missing rather than falling back to this code.

Every function cites the reference file:line it follows.

Pin status (what independent evidence fixes each function):

* ``codebook.lloyd_max_codebook``     pinned: textbook Gaussian Lloyd-Max levels
  (Max 1960), symmetry, Panter-Dite bound, scipy's ``norm.pdf``; exact fp64
  bits against the golden table in ``tests/golden`` when that fixture exists.
* ``quantizer.pack_codes / unpack_codes``   pinned: byte layouts worked out by
  hand from the reference text, round trips for every width.
* ``quantizer.nearest_centroid``      pinned against brute-force argmin; the
  reference's own routine (``kvquant.tq_triton.mse_nearest_centroid``) is not
  shipped, so its behaviour exactly on a midpoint is **parity unpinned**.
* ``quantizer.quantize / dequantize`` pinned: algebraic identities (identity
  rotation, 2-entry codebook = sign quantisation), relative MSE against the
  Lloyd-Max distortion table.
* ``scorer.*``                        pinned: fp64 brute force on tiny inputs,
  closed forms (uniform attention, G=1), scaling invariants, and the reference's
  own outputs in ``tests/golden`` (risk score: 5 cases; expected-attention score
  with the query covariance: 6 cases incl. RoPE on mean and covariance).
  ``scorer.window_attention`` has no counterpart in the reference: **parity
  unpinned** there, pinned by brute force and special cases only.
* ``allocator.optimal_scores_to_bits``  pinned: exhaustive Lagrangian argmin on
  tiny inputs, budget invariants, trivial-case clamps; token choice *inside* a
  group of equal scores at the repair cut-off is implementation-defined in the
  reference (unstable argsort) and therefore **parity unpinned** there.
* ``kvstate.*``                       pinned by tests/test_oracle_kvstate_attention.py:
  every position lands in exactly one level, ``materialize`` equals the
  golden-pinned ``quantizer.dequantize`` at quantised positions, the input at
  16-bit ones and zero at evicted ones, ``materialize_quantized_into`` leaves the
  other two alone, ``truncate`` drops exactly the positions behind the cut,
  ``append_all_exact`` + ``flush_buffer`` re-route exactly the buffered tokens.
* ``attention.decode_attention``      pinned by the same file: equals torch's
  ``scaled_dot_product_attention`` in fp64 (G = 1, 4, 7, with mask and scale),
  returns the value of a single visible token, is invariant under a permutation
  of the tokens, under dropping the evicted ones and under a split of the token
  axis merged by log-sum-exp.
* ``flush.*``                         the decode-time flush scoring; see that
  module's header for its pins.
"""
