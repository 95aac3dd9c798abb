"""CPU-only checks of the C ABI library: it loads, exports every symbol the
headers declare, its tables equal the reference's (SHA-256), and the host-side
error paths (weights parsing) work without a GPU. No compute call is made."""
import ctypes
import hashlib
import os
import re

import numpy as np
import pytest

from lc0_amd import backend as be
from lc0_amd import netgen, netproto

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lc0mi_\w+)\s*\(", text)))


@pytest.mark.parametrize("header", ["lc0mi.h", "lc0mi_kernels.h"])
def test_library_exports_every_declared_symbol(header):
    lib = be.load_library()
    names = _declared_symbols(header)
    assert len(names) >= 8
    for name in names:
        assert hasattr(lib, name), name


def test_tables_match_reference_hashes():
    assert hashlib.sha256(be.attn_policy_map().astype("<i2").tobytes()).hexdigest() == \
        "2cde8db6b669bd5c89646fab72e1572e440dfaaa41c0cab0beba151538398419"
    assert hashlib.sha256(be.conv_policy_map().astype("<i2").tobytes()).hexdigest() == \
        "a65b9ce4b8cf3f99c8a98ad8da746ad09f3397b0ef7271a5dab8bee3cf01c94f"
    assert hashlib.sha256(be.pos_encoding().astype("<f4").tobytes()).hexdigest() == \
        "a6461b73540fadaf6a0480f017077e302d25676521525e6a2f7b32fd5d7dc93d"


def _create_error(buf=None, path=None, opts=b""):
    lib = be.load_library()
    h = ctypes.c_void_p()
    if buf is not None:
        rc = lib.lc0mi_net_create_from_buffer(buf, len(buf), opts, ctypes.byref(h))
    else:
        rc = lib.lc0mi_net_create_from_file(path, opts, ctypes.byref(h))
    msg = lib.lc0mi_last_error().decode()
    if rc == 0:
        lib.lc0mi_net_destroy(h)
    return rc, msg


def test_weight_file_errors_surface_as_messages(tmp_path):
    raw = netproto.serialize_net(netgen.CONFIGS["tiny_attn"]())
    rc, msg = _create_error(buf=raw.replace(b"\xc0\x01\x00\x00", b"\xc1\x01\x00\x00", 1))
    assert rc != 0 and "bad header" in msg
    rc, msg = _create_error(buf=raw[:len(raw) // 2])
    assert rc != 0 and ("truncated" in msg or "Invalid" in msg or "size" in msg)
    rc, msg = _create_error(path=str(tmp_path / "nope.pb.gz").encode())
    assert rc != 0 and "Cannot read weights" in msg
    bad = dict(netgen.CONFIGS["tiny_attn"]())
    bad["min_version"] = {"major": 0, "minor": 99, "patch": 0}
    rc, msg = _create_error(buf=netproto.serialize_net(bad))
    assert rc != 0 and "lc0 version >= 0.99.0 required" in msg
    text = tmp_path / "old.txt.gz"
    import gzip
    with gzip.open(text, "wb") as f:
        f.write(b"2\n1.0 2.0\n")
    rc, msg = _create_error(path=str(text).encode())
    assert rc != 0 and "no longer supported" in msg
    truncated = tmp_path / "trunc.pb.gz"
    good = tmp_path / "good.pb.gz"
    netproto.write_pb_gz(str(good), netgen.CONFIGS["tiny_resnet"](), compresslevel=6)
    truncated.write_bytes(good.read_bytes()[:2000])
    rc, msg = _create_error(path=str(truncated).encode())
    assert rc != 0 and "gzip" in msg
    rpe = netgen.CONFIGS["tiny_attn"]()
    rpe["weights"]["encoder"][0]["mha"]["rpe_q"] = np.zeros(4, np.float32)
    rc, msg = _create_error(buf=netproto.serialize_net(rpe))
    assert rc != 0 and "RPE" in msg
    nohead = netgen.CONFIGS["tiny_resnet"]()
    for k in ("policy", "ip_pol_w", "ip_pol_b"):
        nohead["weights"].pop(k)
    rc, msg = _create_error(buf=netproto.serialize_net(nohead))
    assert rc != 0 and "policy head" in msg


def test_without_a_gpu_creation_fails_loudly():
    """The library never computes on the CPU: with no HIP device the factory
    reports it (on a GPU box the same call succeeds)."""
    import torch
    rc, msg = _create_error(buf=netproto.serialize_net(netgen.CONFIGS["tiny_attn"]()))
    if torch.cuda.is_available():
        assert rc == 0
    else:
        assert rc != 0 and "No HIP device" in msg


def test_null_arguments_are_rejected():
    lib = be.load_library()
    assert lib.lc0mi_net_create_from_buffer(None, 0, b"", None) != 0
    assert lib.lc0mi_comp_compute_blocking(None) != 0
    assert lib.lc0mi_comp_batch_size(None) == 0
    lib.lc0mi_comp_q.restype = ctypes.c_float
    assert np.isnan(lib.lc0mi_comp_q(None, 0))


def test_mutated_weight_files_never_crash_the_loader():
    """Robustness of the wire reader: random byte flips, truncations and length-field corruption of a
    valid net must end in an error return (a parse error, or "No HIP device" when the bytes still
    parse), never in a crash or a hang. Runs without a GPU."""
    import ctypes as C
    import numpy as np
    from lc0_amd import netgen, netproto
    from lc0_amd.backend import load_library
    lib = load_library()
    raw = bytearray(netproto.serialize_net(netgen.CONFIGS["tiny_attn"]()))
    rng = np.random.default_rng(123)
    seen = set()
    for trial in range(400):
        data = bytearray(raw)
        kind = trial % 4
        if kind == 0:      # flip a few bytes anywhere
            for pos in rng.integers(0, len(data), 4):
                data[pos] ^= int(rng.integers(1, 256))
        elif kind == 1:    # truncate
            data = data[:int(rng.integers(0, len(data)))]
        elif kind == 2:    # corrupt bytes near the start (tags and lengths of the outer messages)
            for pos in rng.integers(0, 64, 3):
                data[pos] = int(rng.integers(0, 256))
        else:              # splice a random chunk somewhere
            pos = int(rng.integers(0, len(data)))
            data[pos:pos] = bytes(rng.integers(0, 256, int(rng.integers(1, 40)), dtype=np.uint8))
        buf = (C.c_char * len(data)).from_buffer(data) if len(data) else None
        net = C.c_void_p()
        rc = lib.lc0mi_net_create_from_buffer(buf, len(data), b"", C.byref(net))
        assert rc != 0 and not net.value
        seen.add(lib.lc0mi_last_error().decode(errors="replace")[:40])
    assert len(seen) >= 3, seen      # several distinct failure paths were exercised


@pytest.mark.parametrize("options,message", [
    ("precision=int4", "Precision 'int4' is not supported"),
    ("max_batch=0", "max_batch must be in 1..4096"),
    ("max_batch=5000", "max_batch must be in 1..4096"),
    ("lanes=0", "lanes must be in 1..8"),
    ("lanes=9", "lanes must be in 1..8"),
    ("precision=fp8,fp8_gemms=qkv+nope", "fp8_gemms"),
    ("policy_head=soft", "does not exist in this net"),
    ("value_head=q", "does not exist in this net"),
    ("max_batch=abc", "max_batch"),
    ("mlh=perhaps", "mlh"),
])
def test_option_validation_happens_before_the_device_is_touched(options, message):
    """Backend options are checked while the network is set up, so their error messages can be
    pinned without a GPU (unknown keys are reported after construction, as in lc0,
    src/utils/optionsdict.cc:330-341, and therefore need a device)."""
    from lc0_amd import BackendError, Network, netgen
    with pytest.raises(BackendError, match=message):
        Network(netgen.cached_config("tiny_attn"), options)
