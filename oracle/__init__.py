"""TEST INFRASTRUCTURE: CPU oracle of the BF16 GEMM path (see gemm_oracle.py). Never imported by the product."""
