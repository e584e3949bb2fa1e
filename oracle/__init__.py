"""CPU oracle for the three neural-field hot paths.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is imported by ``tests/``, by ``__graft_entry__.smoke()`` and by
the ``cpu_baseline`` leg of ``bench.py``, where it acts as the checker (or the
timed CPU baseline), never as the product path.

Every function restates, on the CPU with plain torch/numpy, the algorithm of
the reference file:line cited in its docstring.

Pinning status (what independent evidence fixes each function):

* ``hash_encoding.level_resolutions`` / ``level_row_counts`` /
  ``first_hashed_level`` / ``level_row_offsets`` -- pinned by exact rational
  arithmetic (``fractions``) in ``tests/test_oracle_hash.py`` and the golden
  geometry lists stored in ``tests/golden/hash_geometry.json``.
* ``hash_encoding.corner_offsets`` -- pinned by the literal D=2 / D=3 tables of
  ``tests/test_layers/test_hash_encoding.py:40-45`` of the reference.
* ``hash_encoding.corner_rows`` -- pinned by the two literal index tables of
  ``tests/test_layers/test_hash_encoding.py:240-251,285-296`` (dense and
  hashed, T=7), by a Python big-int brute force, and by the range invariant.
* ``hash_encoding.corner_weights`` / ``encode_forward`` -- pinned by the
  reference's corner-pick and mean-of-corners cases
  (``test_hash_encoding.py:109-153``), partition of unity, a constant-table
  closed form and a scalar pure-Python trilinear evaluation.
* ``hash_encoding.encode_backward`` -- pinned against ``torch.autograd``
  through ``encode_forward`` and the per-level column-sum invariant.
* ``mlp.*`` -- pinned against ``torch.nn.Linear`` chains with autograd, the
  reference's own baseline (``tests/test_layers/test_fully_fused_mlp.py:21-35``).
  The 16-bit mode (``round_to=``, ``ste_round``) is pinned separately in
  ``tests/test_oracle_mlp.py``: against ``nn.Linear`` chains whose tensors are
  bfloat16 / float16 under CPU autograd, against a hand-written float64
  back-propagation through the rounded activations, on integer inputs where
  nothing rounds (the mode must be invisible), and on a known answer.
* ``reversible.*`` -- PARITY UNPINNED BY THE REFERENCE (the reference holds no
  reversible MLP).  Pinned only by mathematics: ``inverse(forward(x)) == x`` and
  gradients equal to autograd through the plain composition.  Its 16-bit mode
  (``round_to=``, ``stream_round_every=``) is pinned against a composition with
  the rounding points written out, against couplings of 16-bit ``nn.Linear``
  modules, on integer inputs where nothing rounds, and on a known answer.
"""
