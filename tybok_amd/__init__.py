"""tybok_amd: MI355X (gfx950) kernels for tybok's fp8 action-inference path behind tybok's own
``PolicyEngine`` / ``@register`` plugin API.

Layout:

* ``csrc/``      hand-written HIP kernels + the C ABI (``include/tybok_hip.h``)
* ``native``     ctypes binding of ``libtybok_hip.so``
* ``ops``        tensor-level wrappers (torch = device memory + stream only)
* ``quant``      per-row e4m3fn weight quantisation (the checkpoint-side recipe)
* ``base`` / ``registry`` / ``graph``  the engine API mirrored from the reference
* ``policies/``  SmolVLA- and pi0.5-shaped backends wired to the kernels
"""

__version__ = "0.1.0"
