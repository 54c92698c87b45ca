"""sirius_amd -- the training step that Sirius colocates with inference, native on MI355X.

Only what that one path needs lives here:

* ``csrc/``      hand-written HIP kernels (gfx950) + host runtime + the flat C ABI
* ``_lib``       ctypes binding of ``lib/libtorch_col_hip.so`` (fails loudly when absent)
* ``ops``        tensor-level wrappers over the C ABI (NHWC operators)
* ``resnet``     the ResNet-152 step engine built from those operators
* ``torch_col``  host-side mirror of the reference's ``torch_col`` plugin interface
"""

__version__ = "0.1.0"
