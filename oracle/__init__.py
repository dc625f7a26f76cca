"""CPU oracle for the packed-inference / fused-quantization path.  TEST INFRASTRUCTURE ONLY.

Every function here restates, in numpy (and a little C for the sequential sweeps),
the algorithm of one function of the reference (``/root/reference/src/mlkit``; each
docstring cites the file:line it follows).  Nothing in ``mlkit_amd`` imports this
package: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and only as the checker or the timed CPU baseline.

Pin status (what independently fixes each restatement; tests live in ``tests/``):

* ``bitstream.pack/unpack``         closed form per-bit packer, round trips, known answers
* ``layout.layout_for``             integer table from the reference docs + negative cases
* ``scaling.store_scale``           IEEE conversions (numpy/torch casts as library routine)
* ``scaling.fit_scales/encode``     closed forms, half-step error bound, brute-force argmin
* ``scaling.search_scales``         brute force in float64 at the reference's own tolerance;
                                    exact candidate choice on near ties: **parity unpinned**
* ``scaling.decode_*``              index-map formula restated from the reference's tests
* ``matvec.reconstruct_then_matmul`` definition (dequantise, fp32 matmul)
* ``feedback.coefficients``         inverse-Cholesky identity in float64
* ``feedback.sweep``                classic inverse-Cholesky GPTQ loop (textbook) to 1e-5;
                                    bit-level LDL arithmetic order vs the reference's torch
                                    backend: **parity unpinned** (its block-update GEMM
                                    order is unspecified in the reference as well)
* ``transforms.fwht``               Sylvester matrix product in float64, involution
* ``transforms.paley/factor``       orthogonality, +-1 entries, factor table
* ``transforms.deterministic_signs/layer_seed``  integer hash / sha256 by hand
"""
