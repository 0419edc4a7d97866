"""CPU oracle: TEST INFRASTRUCTURE ONLY.

A plain PyTorch/numpy restatement of the reference's selected-attention hot
path.  Only tests, the smoke check and the benchmark's cpu_baseline leg may
import it; the product package never does.
"""
