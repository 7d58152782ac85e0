"""The in-process fabric between stage engines (threads, mailboxes, failure protocol) on CPU
tensors: no kernel runs here."""
import threading
import time

import pytest
import torch

from bamboo_amd.p2p import (FabricTimeout, LocalFabric, NextStageException, PrevStageException, StageKilled)


def fabric(timeout=5.0):
    return LocalFabric(4, (2, 8, 16), torch.float32, 4, device="cpu", timeout=timeout)


def test_messages_are_keyed_by_batch_and_survive_reading():
    f = fabric()
    a, b = f.endpoint(1), f.endpoint(2)
    a.start_batch(); b.start_batch()
    t = torch.ones(2, 8, 16)
    a.send_activation(0, t, 1)
    assert b.recv_activation(0) is t
    assert b.recv_activation(0) is t                 # not consumed: a replay finds it again
    g = torch.zeros(2, 8, 16)
    b.send_grad(0, g, 2)
    assert a.recv_grad(0, 1) is g
    a.start_batch()                                   # stage 1 moves on; its next message is for batch 1
    a.send_activation(0, t * 2, 1)
    assert torch.equal(b.recv_activation(0), t)       # stage 2 is still in batch 0
    b.start_batch()
    assert torch.equal(b.recv_activation(0), t * 2)
    a.start_batch(); b.start_batch()                  # batch 0 is two behind now: collected
    assert not any(isinstance(k[0], int) and k[0] == 0 for k in f.box)


def test_recv_blocks_until_the_neighbour_sends():
    f = fabric()
    a, b = f.endpoint(1), f.endpoint(2)
    a.start_batch(); b.start_batch()
    got = {}
    th = threading.Thread(target=lambda: got.setdefault("x", b.recv_activation(3)))
    th.start()
    time.sleep(0.2)
    assert "x" not in got
    a.send_activation(3, torch.full((2, 8, 16), 7.0), 1)
    th.join(5)
    assert float(got["x"][0, 0, 0]) == 7.0


def test_timeout_instead_of_hanging():
    f = fabric(timeout=1.0)
    b = f.endpoint(2)
    b.start_batch()
    with pytest.raises(FabricTimeout):
        b.recv_activation(0)


def test_kill_and_three_party_protocol():
    f = fabric()
    pred, victim, succ = f.endpoint(1), f.endpoint(2), f.endpoint(3)
    for e in (pred, victim, succ):
        e.start_batch()
    with pytest.raises(ValueError):
        f.kill(0)
    f.kill(2, at_micro_batch=1)
    pred.send_activation(0, torch.ones(1), 1)
    victim.recv_activation(0)                                    # micro-batch 0 still goes through
    victim.send_activation(0, torch.ones(1), 2)
    with pytest.raises(StageKilled):
        victim.recv_activation(1)
    assert 2 in f.dead
    # both neighbours notice at their next transfer with the dead stage
    with pytest.raises(NextStageException):
        pred.send_activation(1, torch.ones(1), 1)
    assert succ.recv_activation(0) is not None                   # what was sent before stays readable
    with pytest.raises(PrevStageException):
        succ.recv_activation(1)
    with pytest.raises(PrevStageException):
        succ.send_grad(0, torch.ones(1), 3)
    # they agree on the smaller step, whoever reports first
    out = {}
    th = threading.Thread(target=lambda: out.setdefault("succ", succ.coordinate_fail_step(2, 9)))
    th.start()
    time.sleep(0.1)
    assert "succ" not in out                                     # waits for the other report
    assert pred.coordinate_fail_step(2, 6) == 6
    th.join(5)
    assert out["succ"] == 6
    # after the report the survivors wait for the stage to come back instead of failing again
    succ.send_grad(0, torch.ones(1), 3)
    pred.adopt(2)
    assert 2 not in f.dead
    pred.send_activation(1, torch.full((1,), 5.0), 2)            # the predecessor now speaks for stage 2
    assert float(succ.recv_activation(1)) == 5.0
    assert pred.recv_grad(0, 2) is not None                      # and reads what stage 3 sent to stage 2


def test_a_neighbour_that_finished_the_batch_counts_as_reported():
    f = fabric()
    pred, succ = f.endpoint(1), f.endpoint(3)
    pred.start_batch(); succ.start_batch()
    with f.cv:
        f.dead.add(2)
    succ.end_batch([3])
    assert pred.coordinate_fail_step(2, 11) == 11


def test_weights_mailbox():
    f = fabric()
    a, b = f.endpoint(1), f.endpoint(2)
    assert a.recv_weights(2) is None
    msg = {"master": torch.ones(8), "exp_avg": torch.zeros(8), "exp_avg_sq": torch.zeros(8), "step": 3}
    b.send_weights(2, msg)
    assert a.recv_weights(2) is msg


def test_pings_have_a_direction():
    """The lazy schedule's one-element transfers (reference engine.py:1903-1930, 2012-2035): a receive-ping
    reports a dead predecessor as PrevStageException, a send-ping a dead successor as NextStageException,
    and neither reports the neighbour on the other side."""
    f = fabric()
    eps = [f.endpoint(s) for s in range(4)]
    for e in eps:
        e.start_batch()
    for e in eps:                       # everybody alive: silent
        e.ping_prev(e.stage)
        e.ping_next(e.stage)
    with f.cv:
        f.dead.add(2)
    with pytest.raises(PrevStageException):
        eps[3].ping_prev(3)             # stage 3 listens to stage 2
    eps[3].ping_next(3)                 # its successor (the ring closes on stage 0) is fine
    with pytest.raises(NextStageException):
        eps[1].ping_next(1)             # stage 1 sends to stage 2
    eps[1].ping_prev(1)
    eps[0].ping_prev(0)
    eps[0].ping_next(0)
    # once the loss has been reported the pings wait for the adopter like every other transfer
    eps[1].acknowledged.add(2)
    eps[1].ping_next(1)
    with f.cv:
        f.dead.discard(2)
        f.dead.add(3)
    with pytest.raises(PrevStageException):
        eps[0].ping_prev(0)             # the first stage's predecessor in the ring is the last stage
    with pytest.raises(NextStageException):
        eps[2].ping_next(2)
