"""FlexStore as a process of its own: the request loop of the memory manager
behind a transport, and the client end the model runtimes hold.

In the reference the manager's loop (FlexStoreManager.deploy,
muxserve/flexstore/manager.py:747-838) sits behind a ZMQ REP socket and every
runtime process holds a REQ socket (muxserve/zmq_utils.py); both ends exchange
Python objects with send_pyobj / recv_pyobj.  pyzmq is not available to this
build, so the same two methods are provided over the standard library's
multiprocessing.connection (a pickled object per message over a local socket):
PipeServer plays ZMQServer, PipeClient plays ZMQClient, and serve() is the
loop: one request, one reply, requests of all clients answered one at a time
in the order they arrive - which is what serialises the runtimes' allocations
on the one shared KVStorage.

Run as a process:
    python -m muxserve_amd.flexstore_service --address /tmp/fs.sock \
        --num-blocks 4096 --models '{"llama-7b": [32, 32]}' [--log requests.pkl]
"""
import argparse
import json
import pickle
import threading
from multiprocessing.connection import Client, Listener, wait
from typing import Any, List, Optional

from .flexstore import CacheRequestHandler

AUTHKEY = b"muxserve-flexstore"


class PipeServer:
    """The replying end (the role of zmq_utils.ZMQServer with a REP socket):
    recv_pyobj() returns the next request of any connected client, send_pyobj()
    answers that client."""

    def __init__(self, address, authkey: bytes = AUTHKEY):
        self.address = address
        self._listener = Listener(address, authkey=authkey)
        self._conns: List[Any] = []
        self._lock = threading.Lock()
        self._current = None
        self._closed = False
        self._acceptor = threading.Thread(target=self._accept, daemon=True)
        self._acceptor.start()

    def _accept(self):
        while not self._closed:
            try:
                conn = self._listener.accept()
            except (OSError, EOFError):
                return
            with self._lock:
                self._conns.append(conn)

    def recv_pyobj(self, timeout: Optional[float] = None):
        """Blocks until a request arrives (None after `timeout` seconds without one)."""
        waited = 0.0
        while True:
            with self._lock:
                conns = list(self._conns)
            ready = wait(conns, timeout=0.02) if conns else []
            for conn in ready:
                try:
                    req = conn.recv()
                except (EOFError, OSError):          # the client went away
                    with self._lock:
                        self._conns.remove(conn)
                    conn.close()
                    continue
                self._current = conn
                return req
            if not conns:
                threading.Event().wait(0.02)
            waited += 0.02
            if timeout is not None and waited >= timeout:
                return None

    def send_pyobj(self, msg):
        conn, self._current = self._current, None
        if conn is None:
            raise RuntimeError("send_pyobj without a request to answer")
        conn.send(msg)

    def close(self):
        self._closed = True
        try:
            self._listener.close()
        except OSError:
            pass
        with self._lock:
            for conn in self._conns:
                conn.close()
            self._conns.clear()


class PipeClient:
    """The requesting end (the role of zmq_utils.ZMQClient with a REQ socket)."""

    def __init__(self, address, authkey: bytes = AUTHKEY):
        self.address = address
        self._conn = Client(address, authkey=authkey)

    def send_pyobj(self, msg):
        self._conn.send(msg)

    def recv_pyobj(self):
        return self._conn.recv()

    def request(self, req_type: str, req_args=None):
        """One round trip, as the runtimes do it (llm_runtime.py:284-286)."""
        self.send_pyobj((req_type, req_args))
        return self.recv_pyobj()

    def cache_alloc_for(self, model_name: str):
        """The cache_alloc callable prepare_inputs takes, over the transport."""
        return lambda batch_block_request: self.request("cache_alloc", [model_name, batch_block_request])

    def close(self):
        self._conn.close()


def serve(handler: CacheRequestHandler, server: PipeServer, log: Optional[list] = None) -> int:
    """The manager's loop (manager.py:747-838): receive, act, reply, until an
    "exit" request - which, as in the reference, ends the loop without a reply.
    A request the handler raises on ends the loop with that exception, as an
    exception ends the reference's process.  log: optional list that receives
    (request, reply) in the order served.  Returns the number of requests
    answered."""
    served = 0
    while True:
        req = server.recv_pyobj()
        is_exit = isinstance(req, (tuple, list)) and len(req) >= 2 and req[0] == "exit"
        reply = handler.handle(req)
        if log is not None:
            log.append((req, reply))
        if is_exit:
            return served
        server.send_pyobj(reply)
        served += 1


def main(argv=None):
    ap = argparse.ArgumentParser(description="FlexStore request loop over a local socket")
    ap.add_argument("--address", required=True, help="path of the local socket")
    ap.add_argument("--num-blocks", type=int, required=True, help="head-blocks in the pool")
    ap.add_argument("--models", required=True, help='JSON: {"model name": [num_layers, num_heads], ...}')
    ap.add_argument("--num-runtime-processes", type=int, default=1)
    ap.add_argument("--log", default=None, help="pickle the served (request, reply) pairs here on exit")
    args = ap.parse_args(argv)
    from .memory_manager import KVStorage
    handler = CacheRequestHandler(KVStorage(args.num_blocks), {k: tuple(v) for k, v in json.loads(args.models).items()},
                                  args.num_blocks, num_runtime_processes=args.num_runtime_processes)
    server = PipeServer(args.address)
    log: list = []
    try:
        serve(handler, server, log)
    finally:
        server.close()
        if args.log:
            with open(args.log, "wb") as f:
                pickle.dump(log, f)


if __name__ == "__main__":
    main()
