"""An independent Python reading of the reference's model file layout (src/core/serialize.c:6-31,
340-450): used to pin the C loader and to get at a fixture's parameters."""
import struct

import numpy as np

DENSE, LEAKY, ELU, SOFTMAX, LAYERNORM, MHA = 0, 4, 5, 8, 15, 19


def parse_axm(blob):
    """Independent reading of the documented layout: (layers, tensors, stored crc)."""
    off = 0

    def take(fmt):
        nonlocal off
        v = struct.unpack_from("<" + fmt, blob, off)
        off += struct.calcsize("<" + fmt)
        return v if len(v) > 1 else v[0]

    magic, version, n_layers = take("III")
    assert magic == 0x41584F4E and version == 4
    layers = []
    for _ in range(n_layers):
        typ, n_params, n_buffers = take("III")
        extra = None
        if typ == DENSE:
            extra = take("qqB")
        elif typ == LAYERNORM:
            extra = take("qf")
        elif typ in (LEAKY, ELU):
            extra = take("f")
        elif typ == SOFTMAX:
            extra = take("I")
        elif typ == MHA:
            extra = take("qIBB")
        layers.append((typ, n_params, n_buffers, extra))
    tensors = []
    for typ, n_params, n_buffers, _ in layers:
        for _ in range(n_params + n_buffers):
            dtype, ndim = take("II")
            shape = [take("q") for _ in range(ndim)]
            assert dtype == 0
            n = int(np.prod(shape))
            tensors.append(np.frombuffer(blob, "<f4", n, off).reshape(shape))
            off += 4 * n
    crc = take("I")
    assert off == len(blob)
    return layers, tensors, crc
