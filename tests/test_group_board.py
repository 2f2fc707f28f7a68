"""The DP group's shared-memory agreement board: a peer that has exited is noticed at once, also while its parent
has not reaped it yet (a zombie still has a pid)."""
import os
import time
import uuid

import numpy as np
import pytest

from kafka_llm_service_amd.runtime import native


def test_exchange_and_unreaped_peer():
    name = f"/kafka_board_test_{os.getpid()}_{uuid.uuid4().hex[:8]}"
    board = native().GroupBoard(name, 2, 0, True)
    pid = os.fork()
    if pid == 0:  # rank 1: one exchange, then gone without anybody waiting for it
        try:
            peer = native().GroupBoard(name, 2, 1, False)
            peer.exchange(np.asarray([3, 0, 0], dtype=np.int64), 20.0)
        finally:
            os._exit(0)
    try:
        got = board.exchange(np.asarray([1, 5, 0], dtype=np.int64), 20.0)
        assert [int(v) for v in got] == [3, 5, 0]
        time.sleep(0.3)  # the child has exited and is a zombie now (this process has not waited for it)
        t0 = time.monotonic()
        with pytest.raises(RuntimeError, match="gone"):
            board.exchange(np.asarray([1, 1, 0], dtype=np.int64), 20.0)
        assert time.monotonic() - t0 < 5.0
    finally:
        board.unlink()
        os.waitpid(pid, 0)
