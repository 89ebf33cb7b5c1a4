"""TEST INFRASTRUCTURE -- not part of the product.

CPU restatement of dlgrad's generated C kernels and of the Python wrappers that
launch them.  Only tests/, the smoke check and the benchmark's cpu_baseline leg
import this package; nothing under dlgrad_amd/ does.
"""
