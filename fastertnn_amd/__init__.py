"""MI355X (gfx950) implementation of the FasterTNN ternary/binary inference hot path.

The product is ``libftnn_hip.so`` (hand-written HIP kernels behind a C ABI, see
``include/ftnn.h``).  This package only binds that ABI for Python callers:

* ``fastertnn_amd.lib``    -- ctypes binding: device-memory entry points driven with
  torch tensors, and the reference's host-memory entry points driven with numpy.
* ``fastertnn_amd.synth``  -- seeded, bit-reproducible synthetic inputs.
* ``fastertnn_amd.build``  -- in-tree hipcc build of the library.

There is no CPU fallback: importing ``fastertnn_amd.lib`` without the built
library raises.
"""
TNN, TBN, BTN, BNN = 0, 1, 2, 3
TYPE_NAMES = {TNN: "tnn", TBN: "tbn", BTN: "btn", BNN: "bnn"}


def act_is_ternary(t):
    return t in (TNN, TBN)


def weight_is_ternary(t):
    return t in (TNN, BTN)
