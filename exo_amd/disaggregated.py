"""Disaggregated prefill: this engine as the prefill server (or client) of the reference's
KV wire protocol, so that an MI355X can prefill for decoders on other machines.

Wire format (src/exo/worker/disaggregated/protocol.py:12-152, server.py:19-38):
every frame is a 4-byte big-endian length followed by a msgpack map.  The reference
encodes ``msgspec.Struct`` values, which serialise as maps keyed by field name in field
order; tagged variants carry the tag under the key ``"type"`` first.  The request is one
``PrefillRequest`` frame; the reply is one ``Header`` frame, then ``kv_chunk`` /
``arrays_state`` messages, closed by ``done`` (or ``error``).  K and V travel as
``[tokens, heads, head_dim]`` bytes of the header's dtype, positions
``[start_pos, offset)`` of every layer (engines/mlx/disaggregated/adapter.py:86-135).

msgspec itself is not needed: the frames are plain msgpack, written here with the
``msgpack`` package in the same key order and with the same minimal integer / str / bin
encodings.  Decoding accepts keys in any order, ignores unknown keys and fills defaults,
as msgspec's decoders do.
"""

from __future__ import annotations

import socket
import threading
import time
from collections import defaultdict
from collections.abc import Callable
from dataclasses import dataclass, field, fields
import struct
from typing import BinaryIO

import msgpack
import torch

from . import ops
from .cache import ShardKVCache

DTYPES = ("bfloat16", "float16", "float32")
_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}


class ProtocolError(Exception):
    pass


# ------------------------------------------------------------------ message types


@dataclass
class Header:
    request_id: str = ""
    model_id: str = ""
    num_layers: int = 0
    dtype: str = "bfloat16"
    start_pos: int = 0


@dataclass
class TensorBlob:
    dtype: str
    shape: tuple
    data: bytes


@dataclass
class KVChunk:
    layer_idx: int
    num_tokens: int
    n_heads: int
    head_dim: int
    dtype: str
    keys: bytes
    values: bytes
    TAG = "kv_chunk"

    @property
    def shape(self) -> tuple[int, int, int]:
        return (self.num_tokens, self.n_heads, self.head_dim)


@dataclass
class ArraysState:
    layer_idx: int
    arrays: list = field(default_factory=list)
    TAG = "arrays_state"


@dataclass
class Done:
    total_tokens: int
    TAG = "done"


@dataclass
class ErrorMessage:
    code: int
    message: str
    TAG = "error"


@dataclass
class PrefillRequest:
    request_id: str = ""
    model_id: str = ""
    token_ids: list = field(default_factory=list)
    start_pos: int = 0


_MESSAGES = {c.TAG: c for c in (KVChunk, ArraysState, Done, ErrorMessage)}
_MISSING = object()


def _to_map(obj) -> dict:
    out: dict = {}
    tag = getattr(obj, "TAG", None)
    if tag is not None:
        out["type"] = tag
    for f in fields(obj):
        v = getattr(obj, f.name)
        if isinstance(v, list) and v and isinstance(v[0], TensorBlob):
            v = [_to_map(b) for b in v]
        elif isinstance(v, tuple):
            v = list(v)
        out[f.name] = v
    return out


_KINDS = {"int": int, "str": str, "bytes": (bytes, bytearray), "list": list, "tuple": (list, tuple)}


def _from_map(cls, m, what: str):
    if not isinstance(m, dict):
        raise ProtocolError(f"Bad {what}: expected a map, got {type(m).__name__}")
    kw = {}
    for f in fields(cls):
        v = m.get(f.name, _MISSING)
        if v is _MISSING:
            from dataclasses import MISSING
            if f.default is not MISSING:
                v = f.default
            elif f.default_factory is not MISSING:  # type: ignore[misc]
                v = f.default_factory()  # type: ignore[misc]
            else:
                raise ProtocolError(f"Bad {what}: missing field {f.name!r}")
        kind = _KINDS.get(str(f.type).split("[")[0])
        if kind is not None and (not isinstance(v, kind) or isinstance(v, bool)):
            raise ProtocolError(f"Bad {what}: field {f.name!r} has type {type(v).__name__}")
        if f.name == "dtype" and v not in DTYPES:
            raise ProtocolError(f"Bad {what}: dtype {v!r}")
        kw[f.name] = v
    if cls is TensorBlob:
        kw["shape"] = tuple(int(d) for d in kw["shape"])
        kw["data"] = bytes(kw["data"])
    if cls is KVChunk:
        kw["keys"], kw["values"] = bytes(kw["keys"]), bytes(kw["values"])
    if cls is ArraysState:
        kw["arrays"] = [_from_map(TensorBlob, b, "tensor blob") for b in kw["arrays"]]
    return cls(**kw)


def _unpack(payload: bytes, what: str):
    try:
        return msgpack.unpackb(payload, raw=False, strict_map_key=False)
    except Exception as exc:  # msgpack raises several unrelated exception types
        raise ProtocolError(f"Bad {what}: {exc}") from exc


# ------------------------------------------------------------------------- frames


_LEN = struct.Struct(">I")  # frame prefix: payload length, 4 bytes big-endian


def _fill(stream: BinaryIO, want: int) -> bytes:
    """``want`` bytes from a stream whose reads may come back short.  End of stream before
    the first byte gives b"" (the peer closed between frames); end of stream inside the
    block is an error."""
    block = memoryview(bytearray(want))
    have = 0
    while have < want:
        piece = stream.read(want - have)
        if not piece:
            if have:
                raise ConnectionError(f"Connection closed after {have}/{want} bytes")
            return b""
        block[have : have + len(piece)] = piece
        have += len(piece)
    return block.tobytes()


def write_frame(stream: BinaryIO, payload: bytes) -> None:
    """One frame = length prefix + payload (protocol.py:76-79), flushed as a unit."""
    prefix = _LEN.pack(len(payload))
    if len(payload) <= 1 << 16:  # small frames go out in one write call
        stream.write(prefix + payload)
    else:  # KV chunks: no copy of the payload
        stream.write(prefix)
        stream.write(payload)
    stream.flush()


def read_frame(stream: BinaryIO) -> bytes:
    """The next frame's payload, or b"" at a clean end of stream (protocol.py:81-86)."""
    prefix = _fill(stream, _LEN.size)
    if not prefix:
        return b""
    (size,) = _LEN.unpack(prefix)
    return _fill(stream, size) if size else b""


def encode(obj) -> bytes:
    return msgpack.packb(_to_map(obj), use_bin_type=True)


def write_header(stream: BinaryIO, header: Header) -> None:
    write_frame(stream, encode(header))


def read_header(stream: BinaryIO) -> Header:
    payload = read_frame(stream)
    if not payload:
        raise ConnectionError("No header received")
    return _from_map(Header, _unpack(payload, "header"), "header")


def write_message(stream: BinaryIO, msg) -> None:
    write_frame(stream, encode(msg))


def read_message(stream: BinaryIO):
    payload = read_frame(stream)
    if not payload:
        return None
    m = _unpack(payload, "message")
    if not isinstance(m, dict) or m.get("type") not in _MESSAGES:
        raise ProtocolError(f"Bad message: unknown type {m.get('type') if isinstance(m, dict) else m!r}")
    return _from_map(_MESSAGES[m["type"]], m, "message")


def write_kv_chunk(stream: BinaryIO, *, layer_idx: int, num_tokens: int, n_heads: int,
                   head_dim: int, dtype: str, keys: bytes, values: bytes) -> None:
    write_message(stream, KVChunk(layer_idx, num_tokens, n_heads, head_dim, dtype, keys, values))


def write_arrays_state(stream: BinaryIO, layer_idx: int, arrays: list) -> None:
    write_message(stream, ArraysState(layer_idx, arrays))


def write_done(stream: BinaryIO, total_tokens: int) -> None:
    write_message(stream, Done(total_tokens))


def write_error(stream: BinaryIO, code: int, message: str) -> None:
    write_message(stream, ErrorMessage(code, message))


def write_request(stream: BinaryIO, job: PrefillRequest) -> None:
    write_frame(stream, encode(job))


def read_request(stream: BinaryIO) -> PrefillRequest:
    payload = read_frame(stream)
    if not payload:
        raise ConnectionError("No request received")
    req = _from_map(PrefillRequest, _unpack(payload, "request"), "request")
    if not all(isinstance(t, int) and not isinstance(t, bool) for t in req.token_ids):
        raise ProtocolError("Bad request: token_ids must be integers")
    return req


# ------------------------------------------------------------ tensors <-> bytes


def tensor_to_bytes(t: torch.Tensor) -> bytes:
    """Raw little-endian bytes of a bf16/f16/f32 tensor (adapter.py:59-65); the device
    copy lands in pinned host memory allocated for it."""
    if t.dtype not in _TORCH_DTYPE.values():
        raise ValueError(f"Unsupported dtype for wire: {t.dtype}")
    t = t.contiguous()
    raw = t.view(torch.uint8) if t.dtype == torch.float32 else t.view(torch.int16).view(torch.uint8)
    if raw.is_cuda:
        host = torch.empty(raw.shape, dtype=torch.uint8, pin_memory=True)
        host.copy_(raw)  # synchronous device -> pinned host
        raw = host
    return raw.numpy().tobytes()


def bytes_to_tensor(data: bytes, shape: tuple, dtype: str, device="cpu") -> torch.Tensor:
    """adapter.py:68-80."""
    if dtype not in _TORCH_DTYPE:
        raise ValueError(f"Unsupported wire dtype: {dtype!r}")
    td = _TORCH_DTYPE[dtype]
    n = 1
    for d in shape:
        n *= int(d)
    if len(data) != n * torch.empty((), dtype=td).element_size():
        raise ValueError(f"{len(data)} bytes do not fill shape {tuple(shape)} of {dtype}")
    host = torch.frombuffer(bytearray(data), dtype=td).reshape(tuple(shape))
    return host.to(device) if str(device) != "cpu" else host


# ---------------------------------------------------------------- server side


def send_kv_cache(stream: BinaryIO, cache: ShardKVCache, *, row: int = 0, dtype: str = "bfloat16",
                  start_pos: int = 0, max_tokens: int | None = None) -> int:
    """One ``kv_chunk`` per local layer with positions [start_pos, offset) of pool row
    ``row`` (adapter.py:86-135).  Layers whose fill level is not beyond ``start_pos`` send
    nothing.  The [Hkv,S,D] -> [n,Hkv,D] re-layout runs on the GPU; only the wire bytes
    cross PCIe."""
    if dtype != "bfloat16":
        raise ValueError("this engine's KV cache is bfloat16")
    offset = cache.offsets[row]
    if max_tokens is not None:
        offset = min(offset, max_tokens)
    if offset <= start_pos:
        return 0
    n = offset - start_pos
    for layer_idx, (k, v) in enumerate(zip(cache.k, cache.v)):
        k_nhd = ops.kv_export_nhd(k[row], start_pos, n)
        v_nhd = ops.kv_export_nhd(v[row], start_pos, n)
        write_kv_chunk(stream, layer_idx=layer_idx, num_tokens=n, n_heads=k_nhd.shape[1],
                       head_dim=k_nhd.shape[2], dtype=dtype, keys=tensor_to_bytes(k_nhd),
                       values=tensor_to_bytes(v_nhd))
    return n


def write_cache_to_wire(wfile: BinaryIO, cache: ShardKVCache, *, row: int = 0,
                        request_id: str = "", model_id: str = "", start_pos: int = 0) -> int:
    """Header, the chunks, Done (adapter.py:212-233)."""
    write_header(wfile, Header(request_id=request_id, model_id=model_id, num_layers=len(cache),
                               dtype="bfloat16", start_pos=start_pos))
    sent = send_kv_cache(wfile, cache, row=row, dtype="bfloat16", start_pos=start_pos)
    write_done(wfile, sent)
    wfile.flush()
    return sent


def run_prefill_for_request(*, model, kv_prefix_cache, request: PrefillRequest,
                            cache: ShardKVCache, row: int = 0) -> ShardKVCache:
    """Fill pool row ``row`` with the KV of the request's first n-2 tokens, reusing and
    updating the prefix cache (engines/mlx/disaggregated/serve.py:21-93).  The decoder
    that asked feeds the last two prompt tokens itself."""
    from .generate import prefill
    toks = [int(t) for t in request.token_ids]
    n_tokens = len(toks)
    matched_index, prefix_hit_length, remaining = None, 0, toks
    if kv_prefix_cache is not None:
        _, remaining, matched_index, _ = kv_prefix_cache.get_kv_cache(cache, toks, row=row)
        prefix_hit_length = n_tokens - len(remaining)
    else:
        cache.reset(rows=range(row, row + 1))
    target_offset = max(0, n_tokens - 2)
    new_tokens = max(0, target_offset - prefix_hit_length)
    prefill_input = remaining[:new_tokens]
    if prefill_input:
        # prefill() leaves len-1 entries; the reference passes the same slice to its own
        # prefill, which has that property too (serve.py:45-58)
        prefill(model, prefill_input, cache, None, row=row)
    if kv_prefix_cache is not None:
        hit_ratio = prefix_hit_length / n_tokens if n_tokens > 0 else 0.0
        if matched_index is not None and hit_ratio >= 0.5:
            kv_prefix_cache.update_kv_cache(matched_index, toks, cache, row,
                                            restore_pos=prefix_hit_length)
        else:
            kv_prefix_cache.add_kv_cache(toks, cache, row)
    return cache


# ---------------------------------------------------------------- client side


@dataclass
class PrefillResult:
    header: Header
    kv_chunks: dict = field(default_factory=dict)  # layer -> [KVChunk]
    arrays: dict = field(default_factory=dict)
    total_tokens: int = 0


def read_result(stream: BinaryIO, on_header=None, on_kv_chunk=None) -> PrefillResult:
    header = read_header(stream)
    if on_header is not None:
        on_header(header)
    result = PrefillResult(header=header)
    by_layer: dict = defaultdict(list)
    received = 0
    while True:
        msg = read_message(stream)
        if msg is None:
            break
        if isinstance(msg, KVChunk):
            by_layer[msg.layer_idx].append(msg)
            received += 1
            if on_kv_chunk is not None:
                on_kv_chunk(msg, received)
        elif isinstance(msg, ArraysState):
            result.arrays[msg.layer_idx] = msg.arrays
        elif isinstance(msg, Done):
            result.total_tokens = msg.total_tokens
            break
        else:
            raise RuntimeError(f"Prefill server error [{msg.code}]: {msg.message}")
    result.kv_chunks = dict(by_layer)
    return result


def _parse_endpoint(endpoint: str) -> tuple[str, int]:
    if ":" in endpoint:
        host, port = endpoint.rsplit(":", 1)
        return host, int(port)
    raise ValueError(f"Invalid endpoint {endpoint}")


def remote_prefill_fetch(endpoint: str, request: PrefillRequest, on_header=None, on_kv_chunk=None,
                         timeout_secs: float = 60.0) -> PrefillResult:
    """engines/mlx/disaggregated/client.py:50-109."""
    host, port = _parse_endpoint(endpoint)
    sock = socket.create_connection((host, port), timeout=timeout_secs)
    sock.setsockopt(socket.IPPROTO_TCP, socket.TCP_NODELAY, 1)
    sock.setsockopt(socket.SOL_SOCKET, socket.SO_RCVBUF, 4 * 1024 * 1024)
    try:
        wfile = sock.makefile("wb", buffering=256 * 1024)
        write_request(wfile, request)
        return read_result(sock.makefile("rb", buffering=256 * 1024), on_header, on_kv_chunk)
    finally:
        sock.close()


def ingest_into_cache(result: PrefillResult, cache: ShardKVCache, *, row: int = 0,
                      start_pos: int = 0) -> int:
    """Write the received chunks into pool row ``row`` behind its first ``start_pos``
    positions and set the fill level (client.py:112-154).  Returns the final offset."""
    received = max((sum(c.num_tokens for c in chunks) for chunks in result.kv_chunks.values()),
                   default=0)
    final_offset = start_pos + received
    if final_offset > cache.max_seq:
        raise ValueError(f"{final_offset} positions do not fit the cache ({cache.max_seq})")
    dev = cache.k[0].device
    for i in range(len(cache)):
        pos = start_pos
        for c in result.kv_chunks.get(i, []):
            if c.dtype != "bfloat16":
                raise ValueError(f"layer {i}: wire dtype {c.dtype} into a bfloat16 cache")
            k = bytes_to_tensor(c.keys, c.shape, c.dtype, dev)
            v = bytes_to_tensor(c.values, c.shape, c.dtype, dev)
            ops.kv_import_nhd(k, cache.k[i][row], pos)
            ops.kv_import_nhd(v, cache.v[i][row], pos)
            pos += c.num_tokens
    cache.offsets[row] = final_offset
    cache.sync_pos()
    return final_offset


# ---------------------------------------------------------------------- server

ResolveHandler = Callable[[PrefillRequest, BinaryIO], bool]

_SEND_BUFFER_BYTES = 4 << 20  # what the reference asks of the socket (server.py:55-56)


class _SocketOut:
    """Unbuffered binary writer over a connected socket: every write goes out whole and at
    once, so the peer sees each frame as soon as the engine has produced it."""

    def __init__(self, conn: socket.socket) -> None:
        self._conn = conn

    def write(self, data) -> int:
        self._conn.sendall(data)
        return len(data)

    def flush(self) -> None:
        pass


class PrefillServer:
    """TCP front of the prefill service: the interface the reference's runner wires up
    (``PrefillServer(resolve, host, port)``, ``stop()``; src/exo/worker/disaggregated/
    server.py:88-110), on a plain accept loop.

    One thread accepts connections; every connection gets a short-lived thread that reads ONE
    request frame, hands it to ``resolve(request, wfile)`` and closes.  ``resolve`` writes the
    reply stream itself and returns whether it took the request; an engine that is
    single-threaded queues the request for its own thread there and waits.  Status replies
    are a zero-layer header followed by an error frame, as the reference's clients expect:
    400 for an undecodable request, 500 when ``resolve`` raises, 503 when it declines."""

    def __init__(self, resolve: ResolveHandler, host: str, port: int) -> None:
        self.resolve = resolve
        self._sock = socket.create_server((host, port), reuse_port=False)
        self._sock.settimeout(0.2)  # the accept loop looks at the stop flag between waits
        self.server_address = self._sock.getsockname()
        self._stopping = threading.Event()
        self._acceptor: threading.Thread | None = threading.Thread(
            target=self._accept_loop, name="prefill-server", daemon=True)
        self._acceptor.start()

    # -- life cycle
    def _accept_loop(self) -> None:
        while not self._stopping.is_set():
            try:
                conn, _peer = self._sock.accept()
            except socket.timeout:
                continue
            except OSError:
                break  # the listening socket was closed
            threading.Thread(target=self._serve_connection, args=(conn,), name="prefill-conn",
                             daemon=True).start()

    def stop(self) -> None:
        self._stopping.set()
        try:
            self._sock.close()
        finally:
            if self._acceptor is not None:
                self._acceptor.join(timeout=5)
                self._acceptor = None

    # -- one connection
    @staticmethod
    def _reply_status(wfile: BinaryIO, code: int, message: str) -> None:
        """Best effort: the peer may already be gone."""
        try:
            write_header(wfile, Header(num_layers=0, dtype="float32"))
            write_error(wfile, code=code, message=message)
        except (OSError, ValueError):
            pass

    def _serve_connection(self, conn: socket.socket) -> None:
        with conn:
            conn.settimeout(None)
            conn.setsockopt(socket.IPPROTO_TCP, socket.TCP_NODELAY, 1)
            conn.setsockopt(socket.SOL_SOCKET, socket.SO_SNDBUF, _SEND_BUFFER_BYTES)
            rfile, wfile = conn.makefile("rb"), _SocketOut(conn)
            try:
                status: tuple[int, str] | None = None
                try:
                    request = read_request(rfile)
                except ConnectionError:
                    return  # closed without sending a request
                except (ProtocolError, ValueError) as exc:
                    request, status = None, (400, f"Bad request: {exc}")
                if request is not None:
                    try:
                        if not self.resolve(request, wfile):
                            status = (503, f"Prefill not picked up for request_id={request.request_id!r}")
                    except Exception as exc:  # the engine's failure becomes the peer's error frame
                        status = (500, str(exc))
                if status is not None:
                    self._reply_status(wfile, *status)
            finally:
                try:
                    rfile.close()
                except OSError:
                    pass


def remote_prefill(prompt_tokens, cache: ShardKVCache, on_prefill_progress=None, *, endpoint: str,
                   request_id: str, model_id: str, start_pos: int = 0, row: int = 0,
                   ) -> tuple[float, int]:
    """Decoder side (engines/mlx/generator/remote_prefill.py:19-72): send the tokens to
    ``endpoint``, ingest the reply behind the row's first ``start_pos`` positions, report
    progress once per full set of layer chunks.  Returns (tokens_per_sec, tokens
    received)."""
    t0 = time.perf_counter()
    toks = [int(t) for t in prompt_tokens]
    total = len(toks)
    num_layers = 0

    def on_header(h: Header) -> None:
        nonlocal num_layers
        num_layers = h.num_layers

    def on_chunk(_c: KVChunk, received: int) -> None:
        if on_prefill_progress is not None and num_layers > 0 and received % num_layers == 0:
            on_prefill_progress(min(received // num_layers, total), total)

    result = remote_prefill_fetch(endpoint, PrefillRequest(request_id, model_id, toks, start_pos),
                                  on_header=on_header, on_kv_chunk=on_chunk)
    final = ingest_into_cache(result, cache, row=row, start_pos=start_pos)
    num_tokens = final - start_pos
    return num_tokens / max(time.perf_counter() - t0, 0.001), num_tokens
