"""Checkpoint transport for live recovery, with the state packed on the device.

``CheckpointTransport`` is the reference's plugin interface
(torchft/checkpointing.py:34-88) and ``CheckpointServer`` keeps the behaviour of
the reference's HTTP implementation (:110-270): requests block until
``send_checkpoint`` allows a step, a request for another step gets HTTP 400,
``disallow_checkpoint`` re-takes the lock before the optimizer mutates the
state, and ``recv_checkpoint`` raises on time-out.  What changes is the payload:
instead of ``torch.save`` / ``torch.load`` the server gathers the device tensors
into one staging buffer with one kernel launch (torchft_amd.state_pack) and
streams header + payload; the receiver uploads the payload chunk by chunk and
returns tensors that live on its GPU.
"""

from __future__ import annotations

import logging
import socket
import threading
import urllib.request
from abc import ABC, abstractmethod
from contextlib import contextmanager
from datetime import timedelta
from http.server import BaseHTTPRequestHandler, ThreadingHTTPServer
from typing import Dict, Generator, Generic, List, Optional, TypeVar

import torch

from . import state_pack

logger: logging.Logger = logging.getLogger(__name__)

T = TypeVar("T")


class CheckpointTransport(Generic[T], ABC):
    """Moves a state dict from a healthy replica to a recovering one."""

    @abstractmethod
    def metadata(self) -> str:
        """A string the remote transport needs to fetch from this one."""
        ...

    @abstractmethod
    def send_checkpoint(
        self, dst_ranks: List[int], step: int, state_dict: T, timeout: timedelta
    ) -> None:
        """Makes ``state_dict`` of ``step`` available to ``dst_ranks``; may be asynchronous."""
        ...

    def disallow_checkpoint(self) -> None:
        """After this returns the state dict may be mutated: nothing more is read from it."""
        ...

    @abstractmethod
    def recv_checkpoint(self, src_rank: int, metadata: str, step: int, timeout: timedelta) -> T:
        """Fetches the state dict of ``step`` from ``src_rank``."""
        ...

    def shutdown(self, wait: bool = True) -> None:
        """Releases the transport's resources."""


@contextmanager
def _timed_acquire(lock: threading.Lock, timeout: timedelta) -> Generator[None, None, None]:
    """Holds ``lock`` for the block or raises ``TimeoutError`` after ``timeout``."""
    if not lock.acquire(timeout=timeout.total_seconds()):
        raise TimeoutError(f"timed out acquiring lock after {timeout}")
    try:
        yield
    finally:
        lock.release()


def _advertised_host() -> str:
    """The host name peers should use (as in the reference, torchft/checkpointing.py:214-216),
    or ``localhost`` when this machine's own name does not resolve (bare containers)."""
    host = socket.gethostname()
    try:
        socket.getaddrinfo(host, None)
        return host
    except OSError:
        return "localhost"


class _IPv6HTTPServer(ThreadingHTTPServer):
    address_family = socket.AF_INET6
    request_queue_size = 1024


class CheckpointServer(CheckpointTransport[T]):
    """HTTP server that serves the current state dict, packed on the device.

    The pack kernel and the device-to-host copies of a request run on the
    server's own HIP stream, ordered after whatever the training stream had
    enqueued when ``send_checkpoint`` was called, so serving does not serialise
    with the training thread's later work.
    """

    def __init__(
        self,
        timeout: timedelta,
        chunk_bytes: int = state_pack.DEFAULT_CHUNK_BYTES,
        allow_pickle: bool = True,
    ) -> None:
        self._allow_pickle = allow_pickle
        self._checkpoint_lock = threading.Lock()
        self._disallowed = False
        self._step = -1
        self._timeout = timeout
        self._chunk_bytes = chunk_bytes
        self._state_dict: Optional[T] = None
        self._ready: Optional["torch.cuda.Event"] = None
        self._streams: Dict[int, "torch.cuda.Stream"] = {}
        self._staging: Optional[torch.Tensor] = None

        # nothing is served before the first send_checkpoint
        self.disallow_checkpoint()

        server = self

        class RequestHandler(BaseHTTPRequestHandler):
            timeout = server._timeout.total_seconds()  # socket timeout of each request

            def do_GET(self) -> None:
                try:
                    assert self.connection.gettimeout() == self.timeout
                    with _timed_acquire(server._checkpoint_lock, server._timeout):
                        step = server._step
                        if self.path != f"/checkpoint/{step}":
                            self.send_response(400)
                            self.send_header("Content-type", "text/plain")
                            self.end_headers()
                            msg = f"invalid checkpoint requested, serving {step} but got {self.path}"
                            logger.error(msg)
                            self.wfile.write(msg.encode())
                            return
                        self.send_response(200)
                        self.send_header("Content-type", "application/octet-stream")
                        self.end_headers()
                        server._serve_state(self.wfile)
                except Exception as e:
                    logger.exception("Exception in checkpoint server when handling %s: %s", self.path, e)
                    self.send_response(500, str(e))
                    self.end_headers()

            def log_message(self, format: str, *args: object) -> None:  # keep stderr quiet
                logger.debug(format, *args)

        self._server = _IPv6HTTPServer(("", 0), RequestHandler)
        logger.info("Started CheckpointServer on %s...", self.address())
        self._thread = threading.Thread(target=self._serve, daemon=True)
        self._thread.start()

    # -- serving -------------------------------------------------------------
    def _serve(self) -> None:
        try:
            self._server.serve_forever()
        except Exception:
            logger.exception("got exception in checkpoint server")

    def _serve_state(self, wfile) -> None:
        plan = state_pack.plan_pack(self._state_dict)
        if not plan.tensors:
            state_pack.write_packed(state_pack.PackedState(plan, None), wfile)
            return
        device = plan.tensors[0].device
        stream = self._streams.get(device.index)
        if stream is None:
            stream = self._streams[device.index] = torch.cuda.Stream(device=device)
        if self._ready is not None:
            stream.wait_event(self._ready)
        with torch.cuda.stream(stream):
            if (
                self._staging is None
                or self._staging.device != device
                or self._staging.numel() < plan.total_bytes
            ):
                self._staging = torch.empty(plan.total_bytes, dtype=torch.uint8, device=device)
            packed = state_pack.pack(self._state_dict, staging=self._staging)
            state_pack.write_packed(packed, wfile, self._chunk_bytes)
            stream.synchronize()

    # -- fetching ------------------------------------------------------------
    @classmethod
    def load_from_address(cls, address: str, timeout: timedelta, allow_pickle: bool = True) -> T:
        """Fetches and unpacks the state dict served at ``address``; device tensors are
        rebuilt on the current GPU.  Nothing is unpickled unless the sender had to embed a
        leaf that JSON cannot express (``allow_pickle=False`` refuses such a state)."""
        logger.info("fetching checkpoint from %s", address)
        with urllib.request.urlopen(address, timeout=timeout.total_seconds()) as f:
            header, staging = state_pack.read_packed(f, None)
        return state_pack.unpack(header, staging, copy=False, allow_pickle=allow_pickle)

    def address(self) -> str:
        """``http://host:port/checkpoint/``; the step number is appended by the fetcher."""
        port = self._server.socket.getsockname()[1]
        return f"http://{_advertised_host()}:{port}/checkpoint/"

    # -- gate ------------------------------------------------------------------
    def disallow_checkpoint(self) -> None:
        """Blocks requests until the next ``allow_checkpoint``."""
        if not self._disallowed:
            self._disallowed = True
            self._checkpoint_lock.acquire()

    def allow_checkpoint(self, step: int) -> None:
        """Lets requests for ``step`` through."""
        self._step = step
        if self._disallowed:
            self._disallowed = False
            self._checkpoint_lock.release()

    def shutdown(self, wait: bool = True) -> None:
        if not wait:
            # non-blocking shutdown of the socketserver loop
            self._server._BaseServer__shutdown_request = True  # type: ignore[attr-defined]
        if wait:
            self._server.shutdown()
            self._thread.join()

    # -- CheckpointTransport -----------------------------------------------------
    def metadata(self) -> str:
        return self.address()

    def send_checkpoint(
        self, dst_ranks: List[int], step: int, state_dict: T, timeout: timedelta
    ) -> None:
        self._state_dict = state_dict
        if torch.cuda.is_available() and torch.cuda.is_initialized():
            self._ready = torch.cuda.Event()
            self._ready.record()
        self.allow_checkpoint(step)

    def recv_checkpoint(self, src_rank: int, metadata: str, step: int, timeout: timedelta) -> T:
        return self.load_from_address(f"{metadata}{step}", timeout, self._allow_pickle)
