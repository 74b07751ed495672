"""CPU oracle for the block-sparse attention forward path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``hbsattn_amd/`` (the product) imports,
links or executes anything in this package; only ``tests/``, the smoke check in
``__graft_entry__.py`` and the ``cpu_baseline`` leg of ``bench.py`` do, and there
only as the checker / the timed CPU baseline, never as a compute path.

Contents
--------
``dense``   vectorised fp32/fp64 masked-dense restatement (torch CPU ops) of the
            reference's golden implementation, reference ``hbsattn/reference.py:23-107``
            (v1) cross-read against ``hbsattn/reference.py:188-265`` (v3), plus a
            list-based restatement of ``hbsattn/utils.py:7-50`` (block geometry).
``scalar``  ctypes front end of ``scalar.c`` — a plain-C, double-precision,
            loop-per-element restatement of the same semantics that derives the
            block geometry from first principles (it never reads ``cu_*_block``
            arrays), so it also cross-checks ``calculate_blocks``.

How the oracle is pinned (no reference code is imported or executed):
  * ``calculate_blocks``: the worked example the reference documents in
    ``README.md:49-63`` (5 samples, 12 k blocks, last-block sizes 16,13,7,2,7),
    a closed form on uniform lengths and hypothesis-style invariants.
  * attention math: reductions to ``torch.nn.functional.scaled_dot_product_attention``
    (all-true mask; ``is_causal``; bottom-right causal with explicit mask; GQA by
    repeating K/V), ``dense`` against ``scalar`` (two independently written
    restatements, different language, different geometry derivation), and
    invariants (rows with no visible key are exactly 0, cross-sequence mask
    entries are ignored, sequences are independent, mask refinement, ...).
  The reference holds no golden vectors for this path (its tests are unseeded
  and compare implementations against each other), so these checks are what pins
  every function here; see ``tests/test_oracle_*.py``.
"""
