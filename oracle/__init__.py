"""CPU oracle of the quantized-linear specification.

TEST INFRASTRUCTURE ONLY.  Nothing under ``ajllm_amd/`` may import this
package; it exists so that tests, the smoke check and the benchmark's CPU
baseline leg have an independent statement of what the HIP kernels must
compute.
"""
