"""CPU oracle for the quantize/deploy hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory; it exists so that tests, the smoke check and the CPU-baseline leg
of the benchmark have an independent statement of the arithmetic to compare
the HIP kernels with.

Modules
-------
int_quant   integer min/max -> scale/offset -> (fake-)quant arithmetic, a
            re-typing of the reference's eager torch op sequence (each
            function cites the reference lines it follows).
deploy      deploy-buffer construction and the two quantized Linear forwards
            (exact fp64 contractions).
mx          MXFP8-E4M3 / MXFP4-E2M1 block-32 with E8M0 shared scales.
            The reference has no such code: parity unpinned against it; the
            spec is pinned by exhaustive checks against torch's own float8
            cast and by format invariants.
hif8        HiFloat8 value table, brute-force nearest encoder, decoder.
            The reference has no such code: parity unpinned against it; the
            table is pinned by its structural invariants.

Pin status per function is listed at the top of each module.
"""
