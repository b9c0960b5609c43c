"""TEST INFRASTRUCTURE ONLY: CPU oracle for the WebGPT forward path.

Nothing in the product (webgpt_amd/) may import this package. Tests, the smoke
entry and the benchmark's cpu_baseline leg use it as the checker.
"""
