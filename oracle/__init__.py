"""CPU restatements of the reference's polar-key decode path: test infrastructure only.

Imported by tests/, by the smoke check and by the benchmark's CPU-baseline leg; the product
(polarquant_amd) never imports this package.
"""
