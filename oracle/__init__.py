"""CPU oracle for the colocated training step.  TEST INFRASTRUCTURE ONLY.

Nothing under ``oracle/`` is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The product path (``sirius_amd``) never
imports this package and has no CPU fallback.

The reference (SiriusInfTra/Sirius) holds no arithmetic for this path: its
training scripts call torchvision / HuggingFace models, ``nn.CrossEntropyLoss``
and ``torch.optim.SGD`` (train/resnet152.py:22-29,84-91; train/swin_b.py:38-45,
83-95), i.e. PyTorch's CPU kernels are the reference arithmetic.  The modules
here restate it:

* ``nn_ops``    NHWC operator wrappers over ``torch.nn.functional`` on CPU fp32
                (the library routines themselves), pinned by ``brute`` in
                ``tests/test_oracle_pins.py``
* ``brute``     numpy / pure-Python closed forms and brute force on tiny inputs
                (7-loop convolution, fp64 batch statistics, first-maximum argmax,
                logsumexp cross-entropy, scalar SGD recurrence)
* ``resnet``    plain ``torch.nn`` ResNet-152 (Bottleneck [3, 8, 36, 3], stride on
                the 3x3) + the reference's step (scale loss, backward, accumulate,
                SGD) -- parity unpinned by the reference's own tests (it commits no
                vectors); pinned here by parameter count, output shape and the
                operator pins above
* ``host``      pure-Python restatements of the plugin's integer bookkeeping
                (batch distributor, perf model, adjust arithmetic)
"""
