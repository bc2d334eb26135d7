"""Checkpoint transport for live recovery, with the state packed on the device.

``CheckpointTransport`` is the reference's plugin interface
(torchft/checkpointing.py:34-88) and ``CheckpointServer`` keeps the behaviour of
the reference's HTTP implementation (:110-270): requests block until
``send_checkpoint`` allows a step, a request for another step gets HTTP 400,
``disallow_checkpoint`` re-takes the lock before the optimizer mutates the
state, and ``recv_checkpoint`` raises on time-out.  What changes is the payload:
instead of ``torch.save`` / ``torch.load`` the server streams header + packed
payload.  The payload is never materialised as a whole: chunks of 64 MiB are
gathered on the device into a three-slot ring (one launch each), cross PCIe into
pinned memory and go out on the socket, each stage overlapping the next chunk's
(torchft_amd.state_pack.stream_packed).  A receiver may fetch the payload as
several byte ranges over parallel connections (``?part=i&of=n``): one TCP stream
is worth about 5 GB/s between Python endpoints, far below PCIe; it uploads each
range chunk by chunk as it arrives and returns tensors that live on its GPU.
"""

from __future__ import annotations

import logging
import os
import socket
import threading
import urllib.parse
import urllib.request
from abc import ABC, abstractmethod
from contextlib import contextmanager
from datetime import timedelta
from http.server import BaseHTTPRequestHandler, ThreadingHTTPServer
from typing import Generator, Generic, List, Optional, TypeVar

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


def _default_streams() -> int:
    # one TCP stream carries what two copies through the kernel allow one core (8-9 GB/s over
    # loopback); eight of them reach 30 GB/s between two processes, four 26 GB/s
    return max(1, int(os.environ.get("TORCHFT_AMD_CHECKPOINT_STREAMS", "8")))


class CheckpointServer(CheckpointTransport[T]):
    """HTTP server that serves the current state dict, packed on the device.

    The gather kernels and the device-to-host copies of a request run on streams
    of their own (pooled, with their device rings, between requests), ordered after
    whatever the training stream had enqueued when ``send_checkpoint`` was called
    and after nothing else, so serving does not serialise with the training
    thread's later work.  Requests for parts of one payload are served
    concurrently; ``disallow_checkpoint`` closes the gate and waits until the
    requests in flight have stopped reading the state.
    """

    def __init__(
        self,
        timeout: timedelta,
        chunk_bytes: int = state_pack.DEFAULT_CHUNK_BYTES,
        allow_pickle: bool = True,
        fetch_streams: Optional[int] = None,
    ) -> None:
        self._allow_pickle = allow_pickle
        self._checkpoint_lock = threading.Lock()  # the gate: held while serving is disallowed
        self._readers = 0                         # requests currently reading the state
        self._readers_cv = threading.Condition()
        self._disallowed = False
        self._step = -1
        self._timeout = timeout
        self._chunk_bytes = chunk_bytes
        self._fetch_streams = fetch_streams if fetch_streams is not None else _default_streams()
        self._state_dict: Optional[T] = None
        self._plan: Optional[state_pack.PackPlan] = None
        self._ready: Optional["torch.cuda.Event"] = None

        # nothing is served before the first send_checkpoint
        self.disallow_checkpoint()

        server = self

        class RequestHandler(BaseHTTPRequestHandler):
            timeout = server._timeout.total_seconds()  # socket timeout of each request

            def do_GET(self) -> None:
                registered = False
                try:
                    assert self.connection.gettimeout() == self.timeout
                    url = urllib.parse.urlsplit(self.path)
                    with _timed_acquire(server._checkpoint_lock, server._timeout):
                        step = server._step
                        if url.path != f"/checkpoint/{step}":
                            self.send_response(400)
                            self.send_header("Content-type", "text/plain")
                            self.end_headers()
                            msg = f"invalid checkpoint requested, serving {step} but got {self.path}"
                            logger.error(msg)
                            self.wfile.write(msg.encode())
                            return
                        # the gate is open: count this request as a reader, then let other
                        # requests through while it is served
                        with server._readers_cv:
                            server._readers += 1
                        registered = True
                    query = urllib.parse.parse_qs(url.query)
                    part = int(query.get("part", ["0"])[0])
                    parts = int(query.get("of", ["1"])[0])
                    if parts < 1 or not 0 <= part < parts:
                        raise ValueError(f"part {part} of {parts}")
                    self.send_response(200)
                    self.send_header("Content-type", "application/octet-stream")
                    self.end_headers()
                    server._serve_state(self.wfile, part, parts)
                except Exception as e:
                    logger.exception("Exception in checkpoint server when handling %s: %s", self.path, e)
                    try:
                        self.send_response(500, str(e))
                        self.end_headers()
                    except Exception:
                        pass  # the response was already under way
                finally:
                    if registered:
                        with server._readers_cv:
                            server._readers -= 1
                            server._readers_cv.notify_all()

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

    def _serve_state(self, wfile, part: int = 0, parts: int = 1) -> None:
        plan = self._plan
        assert plan is not None, "nothing to serve"
        lo, hi = state_pack.split_range(plan.total_bytes, part, parts)
        if plan.tensors:
            with torch.cuda.device(plan.tensors[0].device):
                state_pack.stream_packed(plan, wfile, lo, hi, self._chunk_bytes, after=self._ready)
        else:
            state_pack.stream_packed(plan, wfile, lo, hi, self._chunk_bytes)

    # -- fetching ------------------------------------------------------------
    @classmethod
    def load_from_address(
        cls, address: str, timeout: timedelta, allow_pickle: bool = True, streams: Optional[int] = None
    ) -> T:
        """Fetches and unpacks the state dict served at ``address``; device tensors are
        rebuilt on the current GPU (as views of one staging buffer that the payload is
        uploaded into).  A payload of more than 256 MiB is fetched as ``streams`` byte
        ranges over parallel connections.  Nothing is unpickled unless the sender had to
        embed a leaf that JSON cannot express (``allow_pickle=False`` refuses such a state)."""
        logger.info("fetching checkpoint from %s", address)
        streams = streams if streams is not None else _default_streams()
        seconds = timeout.total_seconds()
        device = torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else None
        with urllib.request.urlopen(f"{address}?part=0&of={streams}", timeout=seconds) as f:
            header = state_pack.read_header(f)
            total = state_pack.header_total_bytes(header)
            if total == 0 or device is None:
                state_pack.parse_header(header, allow_pickle=False, decode_skeleton=False)
                if total:
                    raise RuntimeError("the packed state holds device tensors and no GPU is visible")
                return state_pack.unpack(header, None, copy=False, allow_pickle=allow_pickle)
            state_pack.check_payload_fits(header, device)
            staging = torch.empty(total, dtype=torch.uint8, device=device)
            torch.cuda.current_stream(device).synchronize()
            errors: List[BaseException] = []

            def fetch_part(part: int) -> None:
                try:
                    with torch.cuda.device(device):
                        lo, hi = state_pack.split_range(total, part, streams)
                        if lo >= hi:
                            return  # a small payload does not fill every range: nothing to ask for
                        with urllib.request.urlopen(f"{address}?part={part}&of={streams}", timeout=seconds) as g:
                            if state_pack.read_header(g) != header:
                                raise RuntimeError("the served state changed between two parts of one fetch")
                            state_pack.read_payload(g, staging, lo, hi)
                except BaseException as e:  # re-raised by the calling thread
                    errors.append(e)

            # ranges 1.. on threads of their own (small payloads: one after the other, here)
            parallel = total > (256 << 20)
            workers = [threading.Thread(target=fetch_part, args=(k,), daemon=True)
                       for k in range(1, streams)] if parallel else []
            for w in workers:
                w.start()
            lo, hi = state_pack.split_range(total, 0, streams)
            state_pack.read_payload(f, staging, lo, hi)
        if not parallel:
            for k in range(1, streams):
                fetch_part(k)
        for w in workers:
            w.join(seconds)
            if w.is_alive():
                raise TimeoutError(f"timed out fetching a part of the checkpoint from {address}")
        if errors:
            raise errors[0]
        return state_pack.unpack(header, staging, copy=False, allow_pickle=allow_pickle)

    def address(self) -> str:
        """``http://host:port/checkpoint/``; the step number is appended by the fetcher."""
        port = self._server.socket.getsockname()[1]
        return f"http://{_advertised_host()}:{port}/checkpoint/"

    # -- gate ------------------------------------------------------------------
    def disallow_checkpoint(self) -> None:
        """Blocks requests until the next ``allow_checkpoint``; returns once no request is
        reading the state any more."""
        if not self._disallowed:
            self._disallowed = True
            self._checkpoint_lock.acquire()
            with self._readers_cv:
                while self._readers:
                    self._readers_cv.wait()

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
        self._plan = state_pack.plan_pack(state_dict)  # walks the dict once, keeps the tensors alive
        if torch.cuda.is_available() and torch.cuda.is_initialized():
            self._ready = torch.cuda.Event()
            self._ready.record()
        self.allow_checkpoint(step)

    def recv_checkpoint(self, src_rank: int, metadata: str, step: int, timeout: timedelta) -> T:
        return self.load_from_address(f"{metadata}{step}", timeout, self._allow_pickle, self._fetch_streams)
