"""CPU oracle: a restatement of the reference's per-rank algorithms.

TEST INFRASTRUCTURE ONLY. Nothing under ``jigsaw_amd/`` imports this package;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and only as the checker / the timed CPU baseline.

Every function cites the reference file:line it follows (paths relative to the
reference checkout, ``jigsaw/...``). The arithmetic the reference delegates to
``torch`` (``F.conv*``, ``torch.nn.grad.conv*``, ``torch.roll``) is called
through the same ``torch`` CPU operators here; jigsaw's own arithmetic (span
integers, copy / add placement and order, the math attention core, the
online-softmax merge, the LayerNorm combine) is restated.

How each part is pinned (see ``tests/test_oracle_*.py``):
  halo.needed_input_span     brute force over (G, n, k, s, p, d) grids
  halo.gather (assemble)     == zero_pad(global)[window], exact, any dtype
  halo.scatter_add (fold)    adjoint identity <Ax, g> == <x, A^T g>; global
                             conv_input identity; order restated with torch add_
  conv fwd/dgrad/wgrad       torch fp64 autograd + 7-loop brute force (tiny)
  attention step / merge     full softmax(QK^T)V over concatenated chunks (fp64);
                             merge special cases (l1=-inf, l1=l2, permutation)
  attention backward         autograd through full attention on concatenated K/V
  layernorm partials         F.layer_norm over the full width + autograd
  roll                       torch.roll on the assembled global tensor, exact
  swin window attention      the block on an undivided image
No function here is "parity unpinned".
"""
