"""Semantic pins of the stage oracle (CPU, tiny shapes): redundant computation changes nothing,
and a stage that absorbed its successor ends with the gradients of own+shadow run as one stage."""
import pytest
import torch

from oracle import layers as ol
from oracle import schedule as osched
from oracle.stage import OraclePeer, OracleStage

CFG = ol.TransformerCfg(hidden=32, heads=4, ffn=64, activation="gelu_tanh", ln="standard", mask="causal")
PARTS = [0, 2, 4, 6, 8]
M, B, SEQ = 4, 2, 8


def make_inputs(seed=0):
    g = torch.Generator().manual_seed(seed)
    acts = [torch.randn(B, SEQ, 32, generator=g, dtype=torch.float64) for _ in range(M)]
    targets = [torch.randn(B, SEQ, 32, generator=g, dtype=torch.float64) for _ in range(M)]
    grads = [torch.randn(B, SEQ, 32, generator=g, dtype=torch.float64) for _ in range(M)]
    return acts, targets, grads


def test_rc_does_not_change_results():
    acts, targets, grads = make_inputs()
    res = []
    for rl, eager in [(0, False), (1, True)]:
        st = OracleStage(CFG, PARTS, 1, M, dtype=torch.float64, redundancy_level=rl, eager=eager)
        peer = OraclePeer(acts, M, grads={1: grads})
        bufs, info = st.run_batch(peer, optimizer_step=False)
        assert info["failed_step"] is None
        res.append((st.named_grads(1), bufs))
    for k in res[0][0]:
        torch.testing.assert_close(res[0][0][k], res[1][0][k], rtol=0, atol=0)
    # redundant outputs == forward of the shadow layers on the own outputs
    st = OracleStage(CFG, PARTS, 1, M, dtype=torch.float64, redundancy_level=1, eager=True)
    bufs = res[1][1]
    for k in range(M):
        ref = st.forward(bufs["out"][(1, k)].detach(), 2)
        torch.testing.assert_close(bufs["out"][(2, k)].detach(), ref, rtol=0, atol=0)


@pytest.mark.parametrize("dead_from", [0, 1, 2, 3])
def test_failover_equals_merged_stage(dead_from):
    """Stage 1 shadows stage 2; stage 2 dies at micro-batch ``dead_from``.  While it lives, the
    gradients it returns are the true ones (computed here from its layers and the MSE head of
    stage 2's output).  After the failover the parameter gradients of both stages must equal
    those of layers 2..5 run as one stage against the same head."""
    acts, targets, _ = make_inputs(1)
    # reference: stages 1+2 fused into one stage (partition [0,2,6,6,8] -> stage 1 owns layers 2..5)
    ref = OracleStage(CFG, [0, 2, 6, 6, 8], 1, M, dtype=torch.float64)
    ref_peer = OraclePeer(acts, M, targets={1: targets})
    ref_bufs, _ = ref.run_batch(ref_peer, optimizer_step=False)
    ref_grads = ref.named_grads(1)

    # the true gradients the live successor would send back for micro-batch k
    succ = OracleStage(CFG, PARTS, 2, M, dtype=torch.float64)
    own_probe = OracleStage(CFG, PARTS, 1, M, dtype=torch.float64)
    true_grads = []
    for k in range(M):
        o1 = own_probe.forward(acts[k], 1).detach().requires_grad_(True)
        o2 = succ.forward(o1, 2)
        (torch.nn.functional.mse_loss(o2, targets[k]) / M).backward()
        true_grads.append(o1.grad)

    st = OracleStage(CFG, PARTS, 1, M, dtype=torch.float64, redundancy_level=1, eager=True)
    peer = OraclePeer(acts, M, grads={1: true_grads}, targets={2: targets})
    peer.dead_from, peer.dead_stage = dead_from, 1
    bufs, info = st.run_batch(peer, optimizer_step=False)
    assert info["failed_step"] is not None and st.stage_ids == [1, 2]
    got = {**st.named_grads(1), **st.named_grads(2)}
    assert set(got) == set(ref_grads)
    for k in ref_grads:
        torch.testing.assert_close(got[k], ref_grads[k], rtol=1e-9, atol=1e-11)
    for k in range(M):
        torch.testing.assert_close(bufs["sent_grad"][(1, k)], ref_bufs["sent_grad"][(1, k)], rtol=1e-9, atol=1e-11)
    assert abs(float(peer.loss) - float(ref_peer.loss)) < 1e-9


@pytest.mark.parametrize("dead_from", [0, 1, 2, 3])
def test_failover_onto_the_last_stage_equals_merged_stage(dead_from):
    """Stage 2 of 4 shadows the LAST stage, which computes the loss from its own labels.  After the last
    stage is lost, stage 2 ends the batch with the gradients and the loss of layers 4..7 run as one last
    stage (3 stages, partition [0, 2, 4, 8]) on the same labels."""
    acts, labels, _ = make_inputs(5)
    ref = OracleStage(CFG, [0, 2, 4, 8], 2, M, dtype=torch.float64)
    ref_peer = OraclePeer(acts, M, labels=labels)
    ref_bufs, _ = ref.run_batch(ref_peer, optimizer_step=False)
    ref_grads = ref.named_grads(2)

    last = OracleStage(CFG, PARTS, 3, M, dtype=torch.float64)
    own_probe = OracleStage(CFG, PARTS, 2, M, dtype=torch.float64)
    true_grads = []
    for k in range(M):
        o1 = own_probe.forward(acts[k], 2).detach().requires_grad_(True)
        (torch.nn.functional.mse_loss(last.forward(o1, 3), labels[k]) / M).backward()
        true_grads.append(o1.grad)

    st = OracleStage(CFG, PARTS, 2, M, dtype=torch.float64, redundancy_level=1, eager=True)
    peer = OraclePeer(acts, M, grads={2: true_grads}, labels=labels)
    peer.dead_from, peer.dead_stage = dead_from, 2
    bufs, info = st.run_batch(peer, optimizer_step=False)
    assert info["failed_step"] is not None and st.stage_ids == [2, 3]
    got = {**st.named_grads(2), **st.named_grads(3)}
    assert set(got) == set(ref_grads)
    for k in ref_grads:
        torch.testing.assert_close(got[k], ref_grads[k], rtol=1e-9, atol=1e-11)
    for k in range(M):
        torch.testing.assert_close(bufs["sent_grad"][(2, k)], ref_bufs["sent_grad"][(2, k)], rtol=1e-9, atol=1e-11)
    assert abs(float(peer.loss) - float(ref_peer.loss)) < 1e-9 and float(peer.loss) > 0


def test_optimizer_step_moves_parameters():
    acts, targets, grads = make_inputs(2)
    st = OracleStage(CFG, PARTS, 1, M, dtype=torch.float32)
    before = {k: v.detach().clone() for k, v in st.named_params(1).items()}
    peer = OraclePeer([a.float() for a in acts], M, grads={1: [g.float() for g in grads]})
    st.run_batch(peer)
    after = st.named_params(1)
    moved = [float((after[k].detach() - before[k]).abs().max()) for k in before]
    # first Adam step moves every touched parameter by ~lr
    assert max(moved) <= 1.01e-3 and min(moved) > 0
