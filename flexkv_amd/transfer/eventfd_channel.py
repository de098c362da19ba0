"""Handing the per-layer eventfds of an inference engine to the layerwise worker.

The engine (consumer) creates ``num_counters x num_layers`` semaphore eventfds
per tensor-parallel rank and passes the descriptors to the worker over a unix
domain socket with SCM_RIGHTS; the worker (server) assembles them into the
``[num_counters, tp_size, num_layers]`` int32 table the transfer group is built
with.  Wire format, as in the reference
(``flexkv/transfer/layerwise.py:51-68, 755-901`` server,
``flexkv/integration/sglang/connector.py:2205-2286`` client):

    client -> server   16 bytes  "iiii": tp_rank, tp_size_per_node, num_layers, num_counters
    client -> server   num_counters messages: payload "i" counter_id,
                       ancillary SCM_RIGHTS with num_layers descriptors
    server -> client   1 byte: 0x01 received, 0x00 failed (client retries)
"""
from __future__ import annotations

import ctypes
import logging
import os
import socket
import struct
import time
from typing import Dict, List, Optional, Sequence

import torch

logger = logging.getLogger("flexkv")

EFD_SEMAPHORE = 0x1
EFD_NONBLOCK = 0x800
_INT = struct.calcsize("i")
_libc = ctypes.CDLL("libc.so.6", use_errno=True)
_libc.eventfd.argtypes = [ctypes.c_uint, ctypes.c_int]
_libc.eventfd.restype = ctypes.c_int


def make_eventfd(semaphore: bool = True, nonblocking: bool = False) -> int:
    flags = (EFD_SEMAPHORE if semaphore else 0) | (EFD_NONBLOCK if nonblocking else 0)
    fd = _libc.eventfd(0, flags)
    if fd < 0:
        err = ctypes.get_errno()
        raise OSError(err, f"eventfd failed: {os.strerror(err)}")
    return fd


def drain_eventfd(fd: int) -> int:
    """Units readable right now from a non-blocking eventfd (semaphore mode: one
    read per unit)."""
    total = 0
    while True:
        try:
            data = os.read(fd, 8)
        except BlockingIOError:
            return total
        if len(data) != 8:
            return total
        total += struct.unpack("Q", data)[0]


def _recv_exact(conn: socket.socket, n: int) -> bytes:
    buf = b""
    while len(buf) < n:
        part = conn.recv(n - len(buf))
        if not part:
            break
        buf += part
    return buf


def _recv_descriptors(conn: socket.socket, count: int):
    payload = bytearray(256)
    nbytes, ancillary, _flags, _addr = conn.recvmsg_into(
        [payload], socket.CMSG_SPACE(count * _INT), 0)
    for level, kind, data in ancillary:
        if level == socket.SOL_SOCKET and kind == socket.SCM_RIGHTS:
            n = len(data) // _INT
            return list(struct.unpack(f"{n}i", data[:n * _INT])), bytes(payload[:nbytes])
    raise RuntimeError("did not receive fds via SCM_RIGHTS")


def receive_layer_eventfds(socket_path: str, tp_group_size: int, num_layers: int,
                           deadline_s: float = 180.0,
                           accept_timeout_s: float = 30.0) -> torch.Tensor:
    """Server side.  Accepts connections until every rank has delivered its
    descriptors or the deadline passes; ranks that never arrive get -1 entries
    (the transfer group skips those).  Returns an empty int32 tensor when nothing
    arrived or the socket could not be set up (eventfd signalling is then off,
    layerwise.py:779-784, 888-892)."""
    def unlink() -> None:
        try:
            os.unlink(socket_path)
        except OSError:
            pass

    unlink()
    server = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
    try:
        server.bind(socket_path)
        server.listen(tp_group_size * 3)  # head-room for clients that retry
        os.chmod(socket_path, 0o777)
    except OSError as e:
        logger.error("[LayerwiseWorker] Failed to bind/listen on %s: %s", socket_path, e)
        server.close()
        return torch.empty(0, dtype=torch.int32)

    by_rank: Dict[int, Dict[int, List[int]]] = {}
    num_counters = 3
    end = time.time() + deadline_s
    try:
        while len(by_rank) < tp_group_size:
            left = end - time.time()
            if left <= 0:
                logger.error("[LayerwiseWorker] Deadline exceeded on %s, received %d/%d ranks",
                             socket_path, len(by_rank), tp_group_size)
                break
            server.settimeout(min(accept_timeout_s, max(left, 0.05)))
            try:
                conn, _ = server.accept()
            except socket.timeout:
                continue
            with conn:
                try:
                    meta = _recv_exact(conn, 16)
                    if len(meta) < 16:
                        raise RuntimeError(f"incomplete metadata: {len(meta)} of 16 bytes")
                    rank, _tp_per_node, layers, counters = struct.unpack("iiii", meta)
                    if not by_rank:
                        num_layers, num_counters = layers, counters
                    sets: Dict[int, List[int]] = {}
                    for _ in range(counters):
                        fds, extra = _recv_descriptors(conn, layers)
                        sets[struct.unpack("i", extra[:4])[0]] = fds
                    by_rank[rank] = sets
                    conn.sendall(b"\x01")
                except Exception as e:  # noqa: BLE001 - the client retries on a NACK
                    logger.warning("[LayerwiseWorker] eventfd reception failed on %s: %s",
                                   socket_path, e)
                    try:
                        conn.sendall(b"\x00")
                    except OSError:
                        pass
    finally:
        server.close()
        unlink()
    if not by_rank:
        return torch.empty(0, dtype=torch.int32)
    table: List[int] = []
    for counter in range(num_counters):
        for rank in range(tp_group_size):
            table.extend(by_rank.get(rank, {}).get(counter, [-1] * num_layers))
    return torch.tensor(table, dtype=torch.int32)


def send_layer_eventfds(socket_path: str, tp_rank: int, tp_size_per_node: int,
                        fds_by_counter: Sequence[Sequence[int]], connect_retries: int = 180,
                        retry_interval_s: float = 1.0, send_retries: int = 3,
                        ack_timeout_s: float = 30.0) -> None:
    """Client side (what an engine's connector does once at start-up)."""
    num_layers = len(fds_by_counter[0])
    last: Optional[BaseException] = None
    for _ in range(send_retries):
        sock: Optional[socket.socket] = None
        try:
            for attempt in range(connect_retries):
                sock = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
                try:
                    sock.connect(socket_path)
                    break
                except (FileNotFoundError, ConnectionRefusedError) as e:
                    sock.close()
                    sock = None
                    if attempt == connect_retries - 1:
                        raise RuntimeError(f"Failed to connect to eventfd socket {socket_path} "
                                           f"after {connect_retries} attempts") from e
                    time.sleep(retry_interval_s)
            sock.sendall(struct.pack("iiii", tp_rank, tp_size_per_node, num_layers,
                                     len(fds_by_counter)))
            for counter_id, fds in enumerate(fds_by_counter):
                rights = struct.pack(f"{len(fds)}i", *fds)
                sock.sendmsg([struct.pack("i", counter_id)],
                             [(socket.SOL_SOCKET, socket.SCM_RIGHTS, rights)])
            sock.settimeout(ack_timeout_s)
            ack = sock.recv(1)
            if ack and ack[0] == 1:
                return
            raise RuntimeError(f"layerwise worker NACK'd eventfd transfer (ack={ack!r})")
        except Exception as e:  # noqa: BLE001
            last = e
            time.sleep(retry_interval_s)
        finally:
            if sock is not None:
                sock.close()
    raise RuntimeError(f"Failed to send eventfds to {socket_path} after {send_retries} "
                       f"attempts: {last}")
