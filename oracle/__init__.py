"""CPU oracle for the HGQ2 quantized-training hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under this directory is part of the shipped
product: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it, and there only as the checker.  The product
package (``hgq2_amd``) never imports it and raises if its HIP library is missing.

Modules
-------
``fixed_point``   eager torch-CPU restatement (one torch op per ``keras.ops`` call)
                  of the stateless fixed-point quantizer that the reference
                  imports from the third-party package ``quantizers>=1.2.2``
                  (reference ``src/hgq/quantizer/internal/fixed_point_quantizer.py:9-10``).
``exact``         integer / rational-arithmetic statement of ``ap_fixed``
                  rounding + overflow and of the minimal-integer-bits rule; used
                  only to pin ``fixed_point`` (it shares no code with it).
``hgq_ref``       eager torch-CPU restatement of the reference's own Python
                  (quantizer classes, QDense, QEinsumDense, ..., EBOPs), autograd backward.
``twin``          builds the ``hgq_ref`` twin of a product layer (same configuration, same variable
                  values) for the parity tests and the ``cpu_baseline`` timings.
"""
