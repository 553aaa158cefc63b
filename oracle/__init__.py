"""CPU oracle for the GEMM path -- TEST INFRASTRUCTURE ONLY.

Importable only from tests/, the smoke check and the benchmark's CPU-baseline leg.
The product package (decx_amd) never imports this.
"""
