"""gpt.rs_amd/blake3.py against the BLAKE3 specification's published known answers, and the parameter ids built on it
(crates/gpt-rs/src/params.rs:29-48)."""
import hashlib

import pytest

from gptrs_amd import models
from gptrs_amd.blake3 import blake3

# digests published with the specification: the empty input, "abc", and the official test-vector inputs (byte i of the
# input is i mod 251) of lengths 1 and 64, 65 (one block exactly, and one byte into the second block of the chunk)
KNOWN = {
    b"": "af1349b9f5f9a1a6a0404dea36dcc9499bcb25c9adc112b7cc9a93cae41f3262",
    b"abc": "6437b3ac38465133ffb63b75273a8db548c558465d79db03fd359c6cd5bd9d85",
    bytes([0]): "2d3adedff11b61f14c886e35afa036736dcd87a74d27b5c1510225d0f592e213",
}


@pytest.mark.parametrize("data,digest", list(KNOWN.items()), ids=["empty", "abc", "one-zero-byte"])
def test_known_answers(data, digest):
    assert blake3(data).hex() == digest


def test_block_boundaries_and_structure():
    """Inputs around the 64-byte block boundary hash to different values, deterministically, and a trailing zero byte is
    not padding (the block length enters the compression)."""
    seen = set()
    for n in (0, 1, 63, 64, 65, 127, 128, 129, 1023, 1024):
        d = blake3(bytes(i % 251 for i in range(n)))
        assert len(d) == 32 and d not in seen and d == blake3(bytes(i % 251 for i in range(n)))
        seen.add(d)
    assert blake3(b"a") != blake3(b"a\0")
    with pytest.raises(ValueError):
        blake3(bytes(1025))


def test_parameter_ids_follow_the_reference_derivation():
    """base id = first 16 bytes of blake3(name), little-endian u128; key = first 16 bytes of
    blake3("gpt-rs:param-key:v1" || namespace u128 LE || base id u128 LE) (params.rs:29-48)."""
    name = "blocks.3.attention.w_qkv"
    base = models.base_param_id(name)
    assert base == int.from_bytes(blake3(name.encode())[:16], "little")
    ns = models.namespace_id("ministral#7")
    key = models.param_id("ministral#7", name)
    want = blake3(b"gpt-rs:param-key:v1" + ns.to_bytes(16, "little") + base.to_bytes(16, "little"))[:16]
    assert key == want and len(key) == 16
    # distinct names and namespaces give distinct keys; the derivation is stable
    assert models.param_id("ministral#7", "lm_head") != key != models.param_id("ministral#8", name)
    assert models.param_id("ministral#7", name) == key
    with pytest.raises(ValueError):
        models.base_param_id("gewicht-ä")     # params.rs:31: names are ASCII
    assert hashlib.blake2b(name.encode(), digest_size=16).digest() != base.to_bytes(16, "little")
