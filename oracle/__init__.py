"""CPU oracle for the gpt-oss layer-kernel path.

TEST INFRASTRUCTURE ONLY. Nothing in the product package may import this
package: it exists so that tests, the smoke check and the benchmark's CPU
baseline can compare the HIP kernels with an independent restatement of the
reference algorithm. See ``oracle/layers.py``.
"""
