"""MI355X (gfx950) backends of awslabs/raf's fused optimizer-step operators.

``raf_amd.op``      imperative ``sgd`` / ``lans`` with the reference's operator signatures
``raf_amd.optim``   ``SGD`` / ``LANS`` optimizer classes with the reference's interface
``raf_amd.kernels`` direct handles on the C ABI (``include/rafhip_optim.h``)
``raf_amd.shapes``  closed-form parameter-shape lists of the benchmark workloads
``raf_amd.build``   in-tree hipcc build of the two shared libraries
"""
__all__ = ["op", "optim", "kernels", "shapes", "build"]
