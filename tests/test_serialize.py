"""Model, tensor and quantized-weight files: the host library against files the reference wrote
(tests/golden/ref_*.axm, ref_tensor.axt), an independent Python reading of the format, and the
crafted inputs of the reference's tests/test_fuzz_serialize.c.  No GPU: tensors live on the CPU
device, nothing is computed."""
import ctypes as C
import os
import struct
import zlib

import numpy as np
import pytest

from axm_format import parse_axm

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")
MODELS = ["mlp", "ffn", "acts", "encoder", "mha_causal"]


@pytest.fixture(scope="module")
def ax():
    from axiom_amd.axiom import Axiom
    a = Axiom()
    a.L.ax_set_default_device(0)
    return a


@pytest.mark.parametrize("tag", MODELS)
def test_reference_model_files_load_and_save_byte_identical(ax, tag, tmp_path):
    L = ax.L
    path = os.path.join(GOLD, f"ref_{tag}.axm")
    blob = open(path, "rb").read()
    layers, tensors, crc = parse_axm(blob)
    assert crc == zlib.crc32(blob[:-4])                       # the checksum is zlib's CRC-32
    model = L.ax_model_load(path.encode())
    assert model, ax.err()
    from axiom_amd.axiom import TP
    params = (TP * 64)()
    net = C.cast(model, C.POINTER(C.c_void_p))[0]             # ax_model_t.net is the first member
    n = L.ax_layer_get_params(net, params, 64)
    assert n == len(tensors)
    for prm, want in zip(params, tensors):
        assert np.array_equal(ax.to_numpy(prm), want)
    out = tmp_path / "again.axm"
    assert L.ax_model_save(model, str(out).encode()) == 0, ax.err()
    assert out.read_bytes() == blob
    L.ax_model_destroy(model)


def test_tensor_file_round_trip(ax, tmp_path):
    L = ax.L
    path = os.path.join(GOLD, "ref_tensor.axt")
    blob = open(path, "rb").read()
    t = L.ax_tensor_load(path.encode())
    assert t, ax.err()
    assert ax.to_numpy(t).shape == (3, 4, 5)
    assert np.array_equal(ax.to_numpy(t).reshape(-1), np.frombuffer(blob, "<f4", 60, 12 + 24))
    out = tmp_path / "t.axt"
    assert L.ax_tensor_save(t, str(out).encode()) == 0 and out.read_bytes() == blob
    ax.free(t)


def test_unsupported_layer_is_refused(ax):
    assert not ax.L.ax_model_load(os.path.join(GOLD, "ref_flatten.axm").encode())
    st, msg = ax.err()
    assert st == 10 and "no forward pass" in msg               # AX_ERR_NOT_IMPLEMENTED


def test_crafted_files_are_rejected(ax, tmp_path):
    """tests/test_fuzz_serialize.c: nothing may crash, everything malformed returns NULL."""
    L = ax.L
    p = tmp_path / "f.axm"
    t = tmp_path / "f.axt"

    def model(data):
        p.write_bytes(data)
        m = L.ax_model_load(str(p).encode())
        if m:
            L.ax_model_destroy(m)
        return bool(m)

    def tensor(data):
        t.write_bytes(data)
        x = L.ax_tensor_load(str(t).encode())
        if x:
            ax.free(x)
        return bool(x)

    assert not model(struct.pack("<I", 0x41584F4E))                                   # truncated header
    assert not model(struct.pack("<III", 0xDEADBEEF, 4, 1))                           # bad magic
    assert not model(struct.pack("<III", 0x41584F4E, 999, 1))                         # future version
    assert not model(struct.pack("<III", 0x41584F4E, 4, 0))                           # no layers
    assert not model(struct.pack("<III", 0x41584F4E, 4, 1 << 30))                     # absurd layer count
    assert not model(b"") and not tensor(b"")
    assert not L.ax_model_load(b"/tmp/ax_does_not_exist_12345.axm")
    assert not L.ax_tensor_load(b"/tmp/ax_does_not_exist_12345.axt")
    garbage = struct.pack("<I", 0x41584F4E) + bytes((i * 37 + 17) & 255 for i in range(4, 4096))
    model(garbage)                                                                    # must not crash
    assert not tensor(struct.pack("<III", 0x41585430, 0, 0xFFFFFFFB))                 # "negative" ndim
    assert not tensor(struct.pack("<IIIqq", 0x41585430, 0, 2, 1 << 40, 1 << 40))      # numel overflow
    assert not tensor(struct.pack("<IIIqq", 0x41585430, 0, 2, -1, 10))                # negative extent
    assert not tensor(struct.pack("<IIIqq", 0x41585430, 0, 2, 10, 10) + b"\0" * 8)    # truncated data
    assert not tensor(struct.pack("<IIIq", 0x41585430, 77, 1, 4) + b"\0" * 16)        # invalid dtype
    # a dense layer whose weight would be enormous must fail before anything is allocated
    assert not model(struct.pack("<IIIIIIqqB", 0x41584F4E, 4, 1, 0, 2, 0, 1 << 40, 1 << 40, 1))
    # every truncation of a good file, and a flipped bit anywhere in it, is rejected
    good = open(os.path.join(GOLD, "ref_mlp.axm"), "rb").read()
    assert model(good)
    for cut in list(range(0, len(good), 37)) + [len(good) - 1]:
        assert not model(good[:cut]), cut
    for pos in range(12, len(good), 101):
        bad = bytearray(good)
        bad[pos] ^= 0x10
        assert not model(bytes(bad)), pos
    # a parameter record with the wrong element count
    layers, tensors, _ = parse_axm(good)
    idx = good.index(struct.pack("<IIqq", 0, 2, 12, 20))
    bad = bytearray(good)
    bad[idx + 8:idx + 16] = struct.pack("<q", 13)
    assert not model(bytes(bad))


def test_quantized_weight_file(ax, tmp_path):
    L = ax.L
    rng = np.random.default_rng(3)
    w = rng.normal(0, 1, (37, 129)).astype(np.float32)
    qw = L.ax_qweight_create_from_fp32(w, 37, 129)
    path = str(tmp_path / "w.axq").encode()
    assert L.ax_qweight_save(qw, path) == 0, ax.err()
    blob = open(path, "rb").read()
    magic, N, K = struct.unpack_from("<Iqq", blob)
    assert (magic, N, K) == (0x41585130, 37, 129) and len(blob) == 20 + 4 * 37 + 37 * 129 + 4
    assert struct.unpack_from("<I", blob, len(blob) - 4)[0] == zlib.crc32(blob[:-4])
    def host_arrays(h):
        d = np.ctypeslib.as_array(C.cast(h.contents.data, C.POINTER(C.c_int8)), (37, 129))
        return d, np.ctypeslib.as_array(C.cast(h.contents.scales, C.POINTER(C.c_float)), (37,))

    q, sc = host_arrays(qw)
    assert np.array_equal(np.frombuffer(blob, "<f4", 37, 20), sc)
    assert np.array_equal(np.frombuffer(blob, "i1", 37 * 129, 20 + 4 * 37).reshape(37, 129), q)
    back = L.ax_qweight_load(path)
    assert back, ax.err()
    assert (back.contents.N, back.contents.K) == (37, 129)
    bq, bsc = host_arrays(back)
    assert np.array_equal(bq, q) and np.array_equal(bsc, sc)
    L.ax_qweight_destroy(back)
    L.ax_qweight_destroy(qw)
    for cut in (0, 3, 19, 100, len(blob) - 1):
        open(path, "wb").write(blob[:cut])
        assert not L.ax_qweight_load(path)
    bad = bytearray(blob)
    bad[200] ^= 1
    open(path, "wb").write(bytes(bad))
    assert not L.ax_qweight_load(path)
    open(path, "wb").write(struct.pack("<Iqq", 0x41585130, 1 << 40, 1 << 40))
    assert not L.ax_qweight_load(path)


def test_reference_loads_what_this_library_saves(ax, tmp_path):
    """A model built here (different shapes from the fixtures) and saved is read back by the
    reference library with identical parameters."""
    from oracle_bind import RefLib, RefTensor, ref_available
    if not ref_available():
        pytest.skip("reference library not built here")
    L = ax.L
    L.ax_set_seed(11)
    seq = L.ax_sequential_create()
    for layer in (L.ax_layernorm_create(10, 1e-5), L.ax_dense_create(10, 14, True), L.ax_gelu_layer_create(),
                  L.ax_dense_create(14, 3, False), L.ax_elu_layer_create(0.5), L.ax_softmax_layer_create(1)):
        assert L.ax_sequential_add(seq, layer)
    model = L.ax_model_create(seq)
    path = str(tmp_path / "mine.axm").encode()
    assert L.ax_model_save(model, path) == 0, ax.err()
    from axiom_amd.axiom import TP
    mine = (TP * 16)()
    n = L.ax_layer_get_params(seq, mine, 16)
    r = RefLib()
    r.L.ax_model_load.restype = C.c_void_p
    r.L.ax_model_load.argtypes = [C.c_char_p]
    r.L.ax_model_destroy.argtypes = [C.c_void_p]
    theirs_model = r.L.ax_model_load(path)
    assert theirs_model
    net = C.cast(theirs_model, C.POINTER(C.c_void_p))[0]
    theirs = (C.POINTER(RefTensor) * 16)()
    assert r.L.ax_layer_get_params(net, theirs, 16) == n == 5
    for a, b in zip(mine[:n], theirs[:n]):
        assert np.array_equal(ax.to_numpy(a), r.numpy(b))
    r.L.ax_model_destroy(theirs_model)
    L.ax_model_destroy(model)
