"""The stats module against the reference's own stats tests (recurrent_drafting/stats_test.py):
step bookkeeping (:23-38), an empty generation's record (:41-50) and the summary of two
generations of three steps with five accepted tokens each, whose acceptance rate the reference
asserts to be exactly 100.0 (:52-72); the other summary fields follow in closed form."""
import pytest

from recurrent_drafting_amd import stats


def test_text_generate_step():
    g = stats.TextGeneration()
    for _ in range(3):
        with g.step() as s:
            assert isinstance(s, stats.TextGeneration.Step)
            with s.time("verify_candidates"):
                pass
            s.set({"input_id_length": 10, "avg_num_accepted": 5})
    assert g.n_steps == 3
    assert g.stats["step"] == [0, 1, 2]
    assert g.stats["input_id_length"] == [10, 10, 10]
    assert g.stats["avg_num_accepted"] == [5, 5, 5]
    assert len(g.stats["wall_times"]["verify_candidates"]) == 3
    assert all(t >= 0 for t in g.stats["wall_times"]["verify_candidates"])


def test_text_generation_posts_its_record():
    ledger = stats.Ledger()
    with stats.text_generation(ledger) as r:
        assert isinstance(r, stats.TextGeneration)
        assert r.n_steps == 0 and len(r.stats["step"]) == 0
    assert ledger.records == [{"step": [], "wall_times": {}}]


def _fake_generate(gr, wall):
    for step in range(3):
        with gr.step() as sr:
            for key in ("generate_candidates", "verify_candidates", "accept_candidate_tokens"):
                with sr.time(key):
                    pass
            sr.set({"input_id_length": 10 + 6 * step, "avg_num_accepted": 5})
    # known durations instead of whatever the clock measured
    for key, seconds in wall.items():
        gr.wall_times[key] = [seconds] * 3


def test_summarize_reference_golden(capsys):
    ledger = stats.Ledger()
    wall = {"generate_candidates": 0.001, "verify_candidates": 0.012, "accept_candidate_tokens": 0.002}
    for _ in range(2):
        with stats.text_generation(ledger) as gr:
            _fake_generate(gr, wall)
    ts, ps = stats.summarize(ledger, 2, 5)
    assert ts.acceptance_rate == 100.0  # the reference's own assertion
    assert ps.acceptance_rate == 100.0
    assert ts.avg_token_per_step == 6.0  # 5 accepted + the LLM's own token, per sequence
    assert ts.avg_generate_candidates == pytest.approx(0.001)
    assert ts.avg_verify_candidates == pytest.approx(0.012)
    assert ts.avg_accept_candidate_tokens == pytest.approx(0.002)
    assert ts.avg_step_time == pytest.approx(0.015)
    assert ts.tokens_per_second == pytest.approx(6.0 / 0.015)  # Tokens/second row of the table
    assert ps.sorted_steps == [0, 1, 2] and ps.sorted_num_tokens_step == [12.0, 12.0, 12.0]
    assert ps.sorted_input_lengths == [10, 16, 22] and ps.sorted_num_tokens_input_length == [12.0, 12.0, 12.0]
    stats.draw_table("candidate_length=5,batch_size=2", ts)
    out = capsys.readouterr().out
    assert "Tokens/second" in out and "400.0000" in out and "100.0000" in out


def test_summarize_ragged_acceptance():
    ledger = stats.Ledger()
    with stats.text_generation(ledger) as gr:
        for accepted in (0.0, 1.5, 4.0):
            with gr.step() as sr:
                for key in ("generate_candidates", "verify_candidates", "accept_candidate_tokens"):
                    with sr.time(key):
                        pass
                sr.set({"input_id_length": 7, "avg_num_accepted": accepted})
    ts, ps = stats.summarize(ledger, 4, 4)
    assert ts.avg_token_per_step == pytest.approx((1 + 2.5 + 5) / 3)
    assert ts.acceptance_rate == pytest.approx(100.0 * ((1 + 2.5 + 5) / 3 - 1) / 4)
    assert ps.sorted_input_lengths == [7] and ps.sorted_num_tokens_input_length == [pytest.approx(4 * (8.5 / 3))]
