"""The closed-loop pipeline model that paces a single real stage (no GPU: the "real" stage is emulated by an
ideal executor here)."""
import pytest

from bamboo_amd.p2p import PipelineClock


def run_real_stage(clock, speed=1.0, extra_after_forward=0.0):
    """Executes the real stage's stream as an ideal in-order executor: a pass starts when the stage is free and
    its receive has arrived, and takes ``speed`` times the model's duration.  Returns (end, busy seconds)."""
    s = clock.sid
    free, busy = 0.0, 0.0
    for kind, k in clock.order[s]:
        arrive = clock.activation_at(k) if kind == "F" else clock.grad_at(k)
        dur = speed * (clock.t_fwd if kind == "F" else clock.t_bwd)
        end = max(free, arrive) + dur
        if kind == "F":
            end += extra_after_forward
            dur += extra_after_forward
        clock.note_done(kind, k, (lambda e=end: e))
        free, busy = end, busy + dur
    return free, busy


@pytest.mark.parametrize("S,sid,M", [(4, 1, 16), (4, 0, 8), (4, 3, 8), (4, 2, 5), (2, 0, 3), (6, 3, 12), (3, 1, 1)])
@pytest.mark.parametrize("tf,tb", [(1.0, 2.0), (1.0, 1.0), (2.0, 3.0)])
def test_balanced_pipeline_closed_form(S, sid, M, tf, tb):
    """Equal stages: the batch takes (M + S - 1)(tf + tb) and every stage idles for (S - 1)(tf + tb) of it,
    the textbook 1F1B figures."""
    c = PipelineClock(S, sid, M, tf, tb)
    end, busy = run_real_stage(c)
    total = (M + S - 1) * (tf + tb)
    assert c.pipeline_end() == pytest.approx(total)
    assert busy == pytest.approx(M * (tf + tb))
    assert total - busy == pytest.approx((S - 1) * (tf + tb))
    # the real stage ends sid backward slots before the pipeline does
    assert end == pytest.approx(total - sid * tb)


def test_deliveries_of_a_middle_stage():
    """S = 4, stage 1, tf = 1, tb = 2, by hand: the first activation arrives after stage 0's first forward (t = 1);
    the first gradient after F0 has gone down two more stages and come back up: own F0 ends at 2, F(2,0) at 3,
    F(3,0) at 4, B(3,0) at 6, B(2,0) at 8 (stage 2 runs its second warm-up forward F(2,1), done at 4, before it)."""
    c = PipelineClock(4, 1, 16, 1.0, 2.0)
    assert c.activation_at(0) == 1.0 and c.activation_at(1) == 2.0 and c.activation_at(2) == 3.0
    c.note_done("F", 0, lambda: 2.0)
    with pytest.raises(RuntimeError):
        c.grad_at(0)                 # stage 2 runs F(2,1) before B(2,0), and own F(1) has not been issued
    c.note_done("F", 1, lambda: 3.0)
    assert c.grad_at(0) == 8.0


def test_a_slow_real_stage_slows_the_pipeline():
    """The loop is closed: a real stage whose passes take 1.25x sets the pace of the whole pipeline."""
    S, sid, M, tf, tb = 4, 1, 16, 1.0, 2.0
    c = PipelineClock(S, sid, M, tf, tb)
    end, busy = run_real_stage(c, speed=1.25)
    assert busy == pytest.approx(1.25 * M * (tf + tb))
    assert c.pipeline_end() >= busy + sid * tf + sid * tb - 1e-9      # own work + fill + drain around it
    assert c.pipeline_end() > (M + S - 1) * (tf + tb) + 0.2 * M * (tf + tb)
    # work appended to every forward (a redundant forward run in line, on the same stream) costs the same way
    c2 = PipelineClock(S, sid, M, tf, tb)
    run_real_stage(c2, extra_after_forward=tf)
    assert c2.pipeline_end() == pytest.approx((M + S - 1) * (tf + tb) + (M - 3) * tf, rel=0.1)


def test_batches_back_to_back():
    """A second batch that starts at the first one's end takes the same time again, on a shifted axis."""
    S, sid, M, tf, tb = 4, 1, 8, 1.0, 2.0
    c = PipelineClock(S, sid, M, tf, tb)
    run_real_stage(c)
    end1 = c.pipeline_end()
    c.start_batch(end1)
    assert c.activation_at(0) == pytest.approx(end1 + sid * tf)
    s = c.sid
    free = end1
    for kind, k in c.order[s]:
        arrive = c.activation_at(k) if kind == "F" else c.grad_at(k)
        end = max(free, arrive) + (tf if kind == "F" else tb)
        c.note_done(kind, k, (lambda e=end: e))
        free = end
    assert c.pipeline_end() == pytest.approx(2 * end1)
