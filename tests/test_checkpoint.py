"""GPTRSCHK v2 checkpoints (docs/formats.md:15-64): the reader against bytes assembled field by field from the
documented layout, the writer against the same bytes, malformed files, and whole models loaded from a checkpoint
through the CPU oracle backend (no GPU needed)."""
import json
import struct

import numpy as np
import pytest

import __graft_entry__ as entry

entry.load_package()
from gptrs_amd import checkpoint as ck_mod  # noqa: E402
from gptrs_amd import models  # noqa: E402
from gptrs_amd.checkpoint import Checkpoint, CheckpointError, write_checkpoint  # noqa: E402
from oracle_backend import OracleBackend  # noqa: E402


def documented_bytes(kind, config, tensors):
    """docs/formats.md: magic, version, config, index (name, base id 0, rank, dims, dtype tag, legacy byte, absolute
    offset, byte length), payloads; tensors in name order as the exporter writes them."""
    cfg = json.dumps({"kind": kind, "config": config}, separators=(",", ":")).encode()
    names = sorted(tensors)
    payloads = [np.ascontiguousarray(tensors[n]).tobytes() for n in names]

    def index(start):
        b = struct.pack("<I", len(names))
        off = start
        for n, p in zip(names, payloads):
            a = tensors[n]
            b += struct.pack("<I", len(n.encode())) + n.encode() + b"\x00" * 16
            b += struct.pack("<I", a.ndim) + b"".join(struct.pack("<Q", d) for d in a.shape)
            b += struct.pack("<I", 0 if a.dtype == np.float32 else 3) + b"\x00" + struct.pack("<QQ", off, len(p))
            off += len(p)
        return b

    n_index = len(index(0))
    start = 8 + 4 + 4 + len(cfg) + 4 + n_index
    return b"GPTRSCHK" + struct.pack("<II", 2, len(cfg)) + cfg + struct.pack("<I", n_index) + index(start) + b"".join(payloads)


TENSORS = {"w.b": np.arange(6, dtype=np.float32).reshape(2, 3), "a": np.array([7, -1, 3], np.int32),
           "scalar": np.array(2.5, np.float32)}
CONFIG = {"vocab_size": 8, "note": "x"}


def test_reader_on_documented_layout(tmp_path):
    path = tmp_path / "m.gptrs"
    path.write_bytes(documented_bytes("gpt", CONFIG, TENSORS))
    with Checkpoint(str(path)) as ck:
        assert ck.kind == "gpt" and ck.config == CONFIG
        assert ck.names() == ["a", "scalar", "w.b"]
        for n, a in TENSORS.items():
            got = ck.array(n)
            assert got.dtype == a.dtype and got.shape == a.shape and np.array_equal(got, a)
        assert ck.entry("w.b").base_id == 0 and ck.entry("a").dtype == "Si32"
        assert "w.b" in ck and "nope" not in ck
        with pytest.raises(CheckpointError, match="not found"):
            ck.array("nope")


def test_writer_emits_documented_layout(tmp_path):
    path = tmp_path / "w.gptrs"
    write_checkpoint(str(path), "gpt", CONFIG, TENSORS)
    assert path.read_bytes() == documented_bytes("gpt", CONFIG, TENSORS)


def test_bf16_payloads_round_trip(tmp_path):
    path = tmp_path / "b.gptrs"
    w = np.random.default_rng(0).normal(size=(5, 4)).astype(np.float32)
    write_checkpoint(str(path), "ministral", {}, {"w": w}, dtypes={"w": "Bf16"})
    from gptrs_amd.ptir import f32_to_bf16_bits
    with Checkpoint(str(path)) as ck:
        assert ck.entry("w").dtype == "Bf16" and ck.entry("w").byte_len == 40
        assert np.array_equal(ck.array("w"), f32_to_bf16_bits(w))


def test_legacy_untagged_config_is_gpt(tmp_path):
    raw = documented_bytes("gpt", CONFIG, TENSORS)
    cfg_new = json.dumps(CONFIG, separators=(",", ":")).encode()
    old_len = struct.unpack_from("<I", raw, 12)[0]
    body = raw[16 + old_len:]
    # offsets move with the config length: rebuild through the writer-independent helper instead
    shift = len(cfg_new) - old_len
    idx_len = struct.unpack_from("<I", body, 0)[0]
    idx = bytearray(body[4:4 + idx_len])
    pos = 4
    for _ in range(struct.unpack_from("<I", idx, 0)[0]):
        nl = struct.unpack_from("<I", idx, pos)[0]
        pos += 4 + nl + 16
        rank = struct.unpack_from("<I", idx, pos)[0]
        pos += 4 + 8 * rank + 4 + 1
        struct.pack_into("<Q", idx, pos, struct.unpack_from("<Q", idx, pos)[0] + shift)
        pos += 16
    path = tmp_path / "legacy.gptrs"
    path.write_bytes(raw[:12] + struct.pack("<I", len(cfg_new)) + cfg_new + struct.pack("<I", idx_len) + bytes(idx) + body[4 + idx_len:])
    with Checkpoint(str(path)) as ck:
        assert ck.kind == "gpt" and ck.config == CONFIG
        assert np.array_equal(ck.array("w.b"), TENSORS["w.b"])


@pytest.mark.parametrize("mutate,msg", [
    (lambda b: b"GPTRSXXX" + b[8:], "magic"),
    (lambda b: b[:8] + struct.pack("<I", 3) + b[12:], "version 3"),
    (lambda b: b[:40], "truncated"),
    (lambda b: b[:-4], "past the end"),
    (lambda b: b"", "magic"),
])
def test_malformed_files_are_rejected(tmp_path, mutate, msg):
    path = tmp_path / "bad.gptrs"
    path.write_bytes(mutate(documented_bytes("gpt", CONFIG, TENSORS)))
    with pytest.raises(CheckpointError, match=msg):
        Checkpoint(str(path))


def test_unknown_dtype_tag_and_length_mismatch(tmp_path):
    raw = bytearray(documented_bytes("gpt", {}, {"a": np.zeros(3, np.float32)}))
    cfg_len = struct.unpack_from("<I", raw, 12)[0]
    entry0 = 16 + cfg_len + 4 + 4            # first index entry
    tag_pos = entry0 + 4 + 1 + 16 + 4 + 8    # name_len, name "a", id, rank, one dim
    bad = bytearray(raw)
    struct.pack_into("<I", bad, tag_pos, 9)
    p = tmp_path / "tag.gptrs"
    p.write_bytes(bytes(bad))
    with pytest.raises(CheckpointError, match="unknown dtype tag 9"):
        Checkpoint(str(p))
    bad = bytearray(raw)
    struct.pack_into("<Q", bad, tag_pos + 4 + 1 + 8, 8)   # byte_len 8 for 3 floats
    p.write_bytes(bytes(bad))
    with pytest.raises(CheckpointError, match="does not match shape"):
        Checkpoint(str(p))


TINY_GPT = models.GptConfig(vocab_size=64, context_length=32, embed_dim=32, num_layers=2, num_heads=4, mlp_ratio=2)
TINY_MINISTRAL = models.MinistralConfig(vocab_size=64, context_length=32, embed_dim=16, num_layers=2, num_heads=4, num_kv_heads=2,
                                        head_dim=4, ffn_dim=48, rotary_dim=4, rope_theta=10000.0)


@pytest.mark.parametrize("cls,cfg,kind,dtype", [(models.Gpt, TINY_GPT, "gpt", "F32"), (models.Ministral, TINY_MINISTRAL, "ministral", "F32"),
                                                (models.Ministral, TINY_MINISTRAL, "ministral", "Bf16")])
def test_model_from_checkpoint_equals_model_in_memory(tmp_path, cls, cfg, kind, dtype):
    be = OracleBackend()
    m = cls.random(cfg, be, seed=4, dtype=dtype, std=0.2)
    path = str(tmp_path / "model.gptrs")
    m.save_checkpoint(path, kind, m.checkpoint_config())
    with Checkpoint(path) as ck:
        assert ck.kind == kind and sorted(ck.names()) == sorted(m.param_names)
        assert ck.entry("lm_head").dtype == dtype
    m2 = cls.from_checkpoint(path, OracleBackend(), dtype=dtype)
    assert m2.config == m.config
    prompt = [3, 17, 42, 5]
    a = models.Generator(m, prompt).generate(6)
    b = models.Generator(m2, prompt).generate(6)
    assert a == b
    for n in m.param_names:
        assert np.array_equal(be.to_numpy(m.param_handle(n)), m2.backend.to_numpy(m2.param_handle(n)))


def test_checkpoint_shape_and_kind_checks(tmp_path):
    be = OracleBackend()
    m = models.Gpt.random(TINY_GPT, be, seed=1, dtype="F32")
    path = str(tmp_path / "g.gptrs")
    m.save_checkpoint(path, "gpt", m.checkpoint_config())
    with pytest.raises(CheckpointError, match="not `ministral`"):
        models.Ministral.from_checkpoint(path, be)
    cfg = dict(m.checkpoint_config(), embed_dim=64)
    m.save_checkpoint(path, "gpt", cfg)
    with pytest.raises(CheckpointError, match="the model expects"):
        models.Gpt.from_checkpoint(path, be)


def test_yarn_config_round_trips(tmp_path):
    from gptrs_amd import functional as F
    cfg = models.MinistralConfig(vocab_size=64, context_length=32, embed_dim=16, num_layers=1, num_heads=4, num_kv_heads=2, head_dim=4,
                                 ffn_dim=48, rotary_dim=4, rope_theta=1e6,
                                 rope_scaling=F.YarnScaling(factor=16.0, original_max_position_embeddings=16384, mscale=1.0, mscale_all_dim=1.0))
    be = OracleBackend()
    m = models.Ministral.random(cfg, be, seed=2, dtype="F32")
    path = str(tmp_path / "y.gptrs")
    m.save_checkpoint(path, "ministral", m.checkpoint_config())
    assert models.Ministral.from_checkpoint(path, OracleBackend(), dtype="F32").config == cfg
