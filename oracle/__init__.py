"""TEST INFRASTRUCTURE ONLY: CPU oracles for the DCNv4 / flash-deformable-attention operators.

Importable only from tests/, the smoke check and the benchmark's CPU-baseline leg.
The dcnv4_amd package never imports this directory.
"""
