"""Wire protocol of disaggregated prefill: framing, message round trips (port of the
reference's src/exo/worker/engines/mlx/disaggregated/tests/test_protocol_roundtrip.py),
hand-assembled msgpack bytes, and the TCP front with a fake resolver.  No GPU."""

import io
import socket
import threading

import pytest

from exo_amd import disaggregated as D


def _mk_bytes(n):
    return bytes(i & 0xFF for i in range(n))


def test_header_roundtrip():
    hdr = D.Header(request_id="r", model_id="m", num_layers=32, dtype="bfloat16", start_pos=42)
    buf = io.BytesIO()
    D.write_header(buf, hdr)
    buf.seek(0)
    got = D.read_header(buf)
    assert got == hdr and got.dtype == "bfloat16" and got.num_layers == 32 and got.start_pos == 42


def test_kv_chunk_roundtrip():
    num_tokens, n_heads, head_dim = 7, 4, 8
    n_bytes = num_tokens * n_heads * head_dim * 2
    keys, values = _mk_bytes(n_bytes), _mk_bytes(n_bytes)[::-1]
    buf = io.BytesIO()
    D.write_kv_chunk(buf, layer_idx=3, num_tokens=num_tokens, n_heads=n_heads, head_dim=head_dim,
                     dtype="bfloat16", keys=keys, values=values)
    buf.seek(0)
    msg = D.read_message(buf)
    assert isinstance(msg, D.KVChunk) and msg.layer_idx == 3
    assert msg.shape == (num_tokens, n_heads, head_dim) and msg.dtype == "bfloat16"
    assert msg.keys == keys and msg.values == values


def test_arrays_state_roundtrip():
    arrs = [D.TensorBlob(dtype="float32", shape=(2, 3), data=_mk_bytes(24)),
            D.TensorBlob(dtype="bfloat16", shape=(5,), data=_mk_bytes(10))]
    buf = io.BytesIO()
    D.write_arrays_state(buf, layer_idx=9, arrays=arrs)
    buf.seek(0)
    msg = D.read_message(buf)
    assert isinstance(msg, D.ArraysState) and msg.layer_idx == 9 and len(msg.arrays) == 2
    assert msg.arrays[0] == arrs[0] and msg.arrays[1] == arrs[1]
    assert msg.arrays[0].shape == (2, 3) and msg.arrays[1].shape == (5,)


def test_done_and_error_roundtrip():
    buf = io.BytesIO()
    D.write_done(buf, 1234)
    D.write_error(buf, code=42, message="boom")
    buf.seek(0)
    m1, m2 = D.read_message(buf), D.read_message(buf)
    assert isinstance(m1, D.Done) and m1.total_tokens == 1234
    assert isinstance(m2, D.ErrorMessage) and (m2.code, m2.message) == (42, "boom")


def test_stream_of_messages():
    hdr = D.Header(num_layers=2, dtype="float32")
    buf = io.BytesIO()
    D.write_header(buf, hdr)
    D.write_kv_chunk(buf, layer_idx=0, num_tokens=1, n_heads=1, head_dim=2, dtype="float32",
                     keys=_mk_bytes(8), values=_mk_bytes(8))
    D.write_arrays_state(buf, 1, [D.TensorBlob("float32", (1,), _mk_bytes(4))])
    D.write_done(buf, total_tokens=1)
    buf.seek(0)
    assert D.read_header(buf) == hdr
    kinds = [type(D.read_message(buf)) for _ in range(3)]
    assert kinds == [D.KVChunk, D.ArraysState, D.Done] and D.read_message(buf) is None


def test_corrupt_message_raises():
    buf = io.BytesIO()
    D.write_header(buf, D.Header(num_layers=1, dtype="float32"))
    buf.write((5).to_bytes(4, "big"))
    buf.write(b"\xff\xff\xff\xff\xff")
    buf.seek(0)
    D.read_header(buf)
    with pytest.raises(D.ProtocolError):
        D.read_message(buf)


def test_truncated_frame_and_bad_fields():
    buf = io.BytesIO((10).to_bytes(4, "big") + b"abc")
    with pytest.raises(ConnectionError):
        D.read_frame(buf)
    assert D.read_frame(io.BytesIO(b"")) == b""
    import msgpack
    bad = msgpack.packb({"type": "done", "total_tokens": "x"})
    with pytest.raises(D.ProtocolError):
        D.read_message(io.BytesIO(len(bad).to_bytes(4, "big") + bad))
    unknown = msgpack.packb({"type": "nope"})
    with pytest.raises(D.ProtocolError):
        D.read_message(io.BytesIO(len(unknown).to_bytes(4, "big") + unknown))
    bad_dtype = msgpack.packb({"num_layers": 1, "dtype": "int8"})
    with pytest.raises(D.ProtocolError):
        D.read_header(io.BytesIO(len(bad_dtype).to_bytes(4, "big") + bad_dtype))


def test_wire_bytes_follow_the_msgpack_layout_of_tagged_structs():
    """Bytes assembled by hand from the msgpack specification: a struct is a map keyed by
    field name in declaration order, a tagged one starts with "type"; integers take their
    shortest form; bytes are bin8/16/32; the frame length is 4 bytes big-endian."""
    def fixstr(s):
        b = s.encode()
        assert len(b) < 32
        return bytes([0xA0 | len(b)]) + b
    done = bytes([0x82]) + fixstr("type") + fixstr("done") + fixstr("total_tokens") + b"\xcd\x04\xd2"
    buf = io.BytesIO()
    D.write_done(buf, 1234)
    assert buf.getvalue() == len(done).to_bytes(4, "big") + done
    hdr = (bytes([0x85]) + fixstr("request_id") + fixstr("r") + fixstr("model_id") + fixstr("m")
           + fixstr("num_layers") + b"\x20" + fixstr("dtype") + fixstr("bfloat16")
           + fixstr("start_pos") + b"\x2a")
    buf = io.BytesIO()
    D.write_header(buf, D.Header("r", "m", 32, "bfloat16", 42))
    assert buf.getvalue() == len(hdr).to_bytes(4, "big") + hdr
    kv = (bytes([0x88]) + fixstr("type") + fixstr("kv_chunk") + fixstr("layer_idx") + b"\x03"
          + fixstr("num_tokens") + b"\x01" + fixstr("n_heads") + b"\x01" + fixstr("head_dim") + b"\x02"
          + fixstr("dtype") + fixstr("bfloat16") + fixstr("keys") + b"\xc4\x04\x00\x01\x02\x03"
          + fixstr("values") + b"\xc4\x04\x03\x02\x01\x00")
    buf = io.BytesIO()
    D.write_kv_chunk(buf, layer_idx=3, num_tokens=1, n_heads=1, head_dim=2, dtype="bfloat16",
                     keys=bytes([0, 1, 2, 3]), values=bytes([3, 2, 1, 0]))
    assert buf.getvalue() == len(kv).to_bytes(4, "big") + kv
    req = (bytes([0x84]) + fixstr("request_id") + fixstr("q") + fixstr("model_id") + fixstr("m")
           + fixstr("token_ids") + b"\x93\x01\xcc\xc8\xce\x00\x01\x86\xa0" + fixstr("start_pos") + b"\x00")
    buf = io.BytesIO()
    D.write_request(buf, D.PrefillRequest("q", "m", [1, 200, 100000], 0))
    assert buf.getvalue() == len(req).to_bytes(4, "big") + req
    buf.seek(0)
    assert D.read_request(buf) == D.PrefillRequest("q", "m", [1, 200, 100000], 0)


def test_decoder_tolerates_key_order_unknown_keys_and_missing_defaults():
    import msgpack
    p = msgpack.packb({"start_pos": 7, "extra": 1, "num_layers": 3})
    h = D.read_header(io.BytesIO(len(p).to_bytes(4, "big") + p))
    assert h == D.Header("", "", 3, "bfloat16", 7)


def test_bytes_tensor_roundtrip():
    import torch
    for dt, name in ((torch.bfloat16, "bfloat16"), (torch.float16, "float16"), (torch.float32, "float32")):
        x = (torch.rand(2, 3, 4) * 10).to(dt)
        y = D.bytes_to_tensor(D.tensor_to_bytes(x), (2, 3, 4), name)
        assert y.dtype == dt and torch.equal(x.view(torch.uint8), y.view(torch.uint8))
    with pytest.raises(ValueError):
        D.bytes_to_tensor(b"\0" * 7, (2, 2), "bfloat16")


def test_tcp_server_paths():
    """server.py:47-86: a resolver that serves, one that declines (503), one that raises
    (500), and an undecodable request (400)."""
    mode = {"v": "ok"}

    def resolve(job, wfile):
        if mode["v"] == "raise":
            raise RuntimeError("kaput")
        if mode["v"] == "decline":
            return False
        D.write_header(wfile, D.Header(job.request_id, job.model_id, 1, "bfloat16", job.start_pos))
        D.write_kv_chunk(wfile, layer_idx=0, num_tokens=len(job.token_ids), n_heads=1, head_dim=1,
                         dtype="bfloat16", keys=b"\0\0" * len(job.token_ids),
                         values=b"\1\1" * len(job.token_ids))
        D.write_done(wfile, len(job.token_ids))
        return True

    srv = D.PrefillServer(resolve, "127.0.0.1", 0)
    try:
        ep = f"127.0.0.1:{srv.server_address[1]}"
        seen = []
        res = D.remote_prefill_fetch(ep, D.PrefillRequest("a", "m", [5, 6, 7], 0),
                                     on_header=lambda h: seen.append(h.num_layers),
                                     on_kv_chunk=lambda c, n: seen.append((c.num_tokens, n)))
        assert res.total_tokens == 3 and res.header.request_id == "a" and seen == [1, (3, 1)]
        assert res.kv_chunks[0][0].values == b"\1\1" * 3
        mode["v"] = "decline"
        with pytest.raises(RuntimeError, match=r"\[503\]"):
            D.remote_prefill_fetch(ep, D.PrefillRequest("b", "m", [1], 0))
        mode["v"] = "raise"
        with pytest.raises(RuntimeError, match=r"\[500\]: kaput"):
            D.remote_prefill_fetch(ep, D.PrefillRequest("c", "m", [1], 0))
        s = socket.create_connection(("127.0.0.1", srv.server_address[1]), timeout=10)
        f = s.makefile("rwb")
        D.write_frame(f, b"\xff\xff\xff")
        hdr = D.read_header(f)
        err = D.read_message(f)
        s.close()
        assert hdr.num_layers == 0 and isinstance(err, D.ErrorMessage) and err.code == 400
    finally:
        srv.stop()
    assert not any(t.name == "prefill-server" and t.is_alive() for t in threading.enumerate())
    with pytest.raises(ValueError):
        D._parse_endpoint("nohost")
