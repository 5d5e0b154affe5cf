"""KV snapshot wire format of an MLA layer: the CPU restatement (oracle/wire.py) against bytes laid out by hand from the
reference's writer, and the library's host-side writer / reader (C ABI, no GPU involved) against the restatement."""
import ctypes as C

import numpy as np
import pytest

from oracle import wire


def u64(v):
    return int(v).to_bytes(8, "little")


def test_restatement_lays_out_the_reference_test_record_by_hand():
    """The record of the reference's session-snapshot test (src/runtime/glm52/rocm_swap.rs:1337): rows 3, interleaved
    pair, 2 latent columns in bf16 mode (group 0, no scales), 1 rope column.  Expected bytes follow write_mla_layer
    (rocm_swap.rs:1090-1113) field by field."""
    record = wire.MlaLayerSerde(3, "InterleavedPair", 2, 1, 0, bytes([1] * 12), None, bytes([2] * 6))
    want = u64(3) + b"\x03" + u64(2) + u64(1) + u64(0) + u64(12) + bytes([1] * 12) + b"\x00" + u64(6) + bytes([2] * 6)
    got = wire.write_mla_layer(record)
    assert got == want and len(got) == 8 + 1 + 24 + 8 + 12 + 1 + 8 + 6
    back, used = wire.read_mla_layer(got + b"tail")
    assert back == record and used == len(want)


def test_restatement_q8_record_and_reader_errors():
    rng = np.random.default_rng(0)
    rows, cols, rope, group = 5, 128, 16, 64
    record = wire.MlaLayerSerde(rows, "BlockParity(1)", cols, rope, group, rng.bytes(rows * cols),
                                rng.bytes(rows * (cols // group) * 2), rng.bytes(rows * rope * 2))
    data = wire.write_mla_layer(record)
    assert data[8] == 2 and data[33 + 8 + rows * cols] == 1  # ownership byte, scales flag
    assert wire.read_mla_layer(data)[0] == record
    with pytest.raises(ValueError, match="truncated"):
        wire.read_mla_layer(data[:-1])
    bad = bytearray(data)
    bad[8] = 9
    with pytest.raises(ValueError, match="ownership"):
        wire.read_mla_layer(bytes(bad))
    bad = bytearray(data)
    bad[33 + 8 + rows * cols] = 7
    with pytest.raises(ValueError, match="flag"):
        wire.read_mla_layer(bytes(bad))


def _record_struct(capi, record, keep):
    def host(data):
        if data is None:
            return None, 0
        buf = (C.c_uint8 * max(len(data), 1)).from_buffer_copy(data if data else b"\x00")
        keep.append(buf)
        return C.cast(buf, C.c_void_p), len(data)

    rec = capi.MlaLayerRecord()
    rec.rows, rec.ownership = record.rows, wire.OWNERSHIP[record.ownership]
    rec.latent_cols, rec.rope_cols, rec.latent_group_size = record.latent_cols, record.rope_cols, record.latent_group_size
    rec.latent, rec.latent_bytes = host(record.latent)
    rec.latent_scales, rec.latent_scales_bytes = host(record.latent_scales)
    rec.rope, rec.rope_bytes = host(record.rope)
    return rec


@pytest.mark.parametrize("kind", ["bf16", "q8", "empty"])
def test_library_writer_and_reader_match_the_restatement(kind):
    from zllm_amd import capi

    lib = capi.load()
    rng = np.random.default_rng(3)
    if kind == "bf16":
        record = wire.MlaLayerSerde(3, "InterleavedPair", 2, 1, 0, bytes([1] * 12), None, bytes([2] * 6))
    elif kind == "q8":
        record = wire.MlaLayerSerde(70, "Full", 512, 64, 64, rng.bytes(70 * 512), rng.bytes(70 * 8 * 2), rng.bytes(70 * 64 * 2))
    else:
        record = wire.MlaLayerSerde(0, "BlockParity(0)", 512, 64, 64, b"", b"", b"")
    keep = []
    rec = _record_struct(capi, record, keep)
    want = wire.write_mla_layer(record)
    assert lib.zllm_kv_mla_layer_wire_bytes(C.byref(rec)) == len(want)
    out = (C.c_uint8 * (len(want) + 16))()
    written = C.c_uint64(0)
    assert lib.zllm_kv_mla_layer_write(C.byref(rec), C.cast(out, C.c_void_p), len(out), C.byref(written)) == 0
    assert written.value == len(want) and bytes(out[: len(want)]) == want
    assert lib.zllm_kv_mla_layer_write(C.byref(rec), C.cast(out, C.c_void_p), len(want) - 1, C.byref(written)) == -1
    # reader: pointers into the buffer, lengths and fields as written
    parsed = capi.MlaLayerRecord()
    used = C.c_uint64(0)
    src = (C.c_uint8 * (len(want) + 3)).from_buffer_copy(want + b"xyz")
    assert lib.zllm_kv_mla_layer_read(C.cast(src, C.c_void_p), len(src), C.byref(parsed), C.byref(used)) == 0
    assert used.value == len(want)
    assert (parsed.rows, parsed.ownership, parsed.latent_cols, parsed.rope_cols, parsed.latent_group_size) == (
        record.rows, wire.OWNERSHIP[record.ownership], record.latent_cols, record.rope_cols, record.latent_group_size)
    assert C.string_at(parsed.latent, parsed.latent_bytes) == record.latent
    assert C.string_at(parsed.rope, parsed.rope_bytes) == record.rope
    if record.latent_scales is None:
        assert not parsed.latent_scales
    else:
        assert C.string_at(parsed.latent_scales, parsed.latent_scales_bytes) == record.latent_scales
    # truncated input and a malformed flag are refused, as by the reference's reader
    assert lib.zllm_kv_mla_layer_read(C.cast(src, C.c_void_p), len(want) - 1, C.byref(parsed), C.byref(used)) == -1


def test_library_refuses_records_whose_lengths_do_not_match_their_shape():
    from zllm_amd import capi

    lib = capi.load()
    keep = []
    record = wire.MlaLayerSerde(4, "Full", 128, 16, 64, b"\x00" * (4 * 128), b"\x00" * (4 * 2 * 2), b"\x00" * (4 * 16 * 2 - 2))
    rec = _record_struct(capi, record, keep)
    assert lib.zllm_kv_mla_layer_wire_bytes(C.byref(rec)) == 0
    data = wire.write_mla_layer(record)  # the restatement writes what it is given; the library's reader flags it
    parsed, used = capi.MlaLayerRecord(), C.c_uint64(0)
    src = (C.c_uint8 * len(data)).from_buffer_copy(data)
    assert lib.zllm_kv_mla_layer_read(C.cast(src, C.c_void_p), len(src), C.byref(parsed), C.byref(used)) == -2
