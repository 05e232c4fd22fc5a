"""BLAKE3 for inputs of at most one chunk (1024 bytes), in pure Python.

The reference derives its stable parameter ids with the `blake3` crate
(crates/gpt-rs/src/params.rs:29-48: `base_param_id` = the first 16 bytes of blake3(name) as a little-endian u128,
`param_key` = the same of blake3("gpt-rs:param-key:v1" || namespace || base id)); neither input reaches 100 bytes, so the
tree mode of the hash (chunks of 1024 bytes combined by parent nodes) never comes into play and is not implemented:
longer inputs raise.  Written from the published specification (BLAKE3 paper, section 2: the compression function is
ChaCha-like over a 4 x 4 state of 32-bit words, seven rounds, message words permuted between rounds); pinned by the
specification's known-answer digests in tests/test_blake3.py.
"""
from __future__ import annotations

import struct

IV = (0x6A09E667, 0xBB67AE85, 0x3C6EF372, 0xA54FF53A, 0x510E527F, 0x9B05688C, 0x1F83D9AB, 0x5BE0CD19)
MSG_PERMUTATION = (2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8)
CHUNK_START, CHUNK_END, ROOT = 1, 2, 8
BLOCK_LEN, CHUNK_LEN = 64, 1024
M32 = 0xFFFFFFFF


def _rotr(x: int, n: int) -> int:
    return ((x >> n) | (x << (32 - n))) & M32


def _g(s, a, b, c, d, mx, my):
    s[a] = (s[a] + s[b] + mx) & M32
    s[d] = _rotr(s[d] ^ s[a], 16)
    s[c] = (s[c] + s[d]) & M32
    s[b] = _rotr(s[b] ^ s[c], 12)
    s[a] = (s[a] + s[b] + my) & M32
    s[d] = _rotr(s[d] ^ s[a], 8)
    s[c] = (s[c] + s[d]) & M32
    s[b] = _rotr(s[b] ^ s[c], 7)


def compress(cv, block_words, counter: int, block_len: int, flags: int):
    """The compression function: 16 output words (the first 8 are the new chaining value)."""
    s = list(cv) + list(IV[:4]) + [counter & M32, (counter >> 32) & M32, block_len, flags]
    m = list(block_words)
    for rnd in range(7):
        _g(s, 0, 4, 8, 12, m[0], m[1])
        _g(s, 1, 5, 9, 13, m[2], m[3])
        _g(s, 2, 6, 10, 14, m[4], m[5])
        _g(s, 3, 7, 11, 15, m[6], m[7])
        _g(s, 0, 5, 10, 15, m[8], m[9])
        _g(s, 1, 6, 11, 12, m[10], m[11])
        _g(s, 2, 7, 8, 13, m[12], m[13])
        _g(s, 3, 4, 9, 14, m[14], m[15])
        if rnd < 6:
            m = [m[p] for p in MSG_PERMUTATION]
    for i in range(8):
        s[i] ^= s[i + 8]
        s[i + 8] ^= cv[i]
    return s


def blake3(data: bytes) -> bytes:
    """The 32-byte digest of `data` (default hash mode, no key), for inputs of one chunk."""
    data = bytes(data)
    if len(data) > CHUNK_LEN:
        raise ValueError("this implementation hashes single chunks (at most 1024 bytes)")
    blocks = [data[i:i + BLOCK_LEN] for i in range(0, len(data), BLOCK_LEN)] or [b""]
    cv = list(IV)
    for i, blk in enumerate(blocks):
        flags = (CHUNK_START if i == 0 else 0) | ((CHUNK_END | ROOT) if i == len(blocks) - 1 else 0)
        words = struct.unpack("<16I", blk.ljust(BLOCK_LEN, b"\0"))
        out = compress(cv, words, 0, len(blk), flags)
        cv = out[:8]
    return struct.pack("<8I", *cv)
