"""Example building pinned by the reference's own vectors (ferrotensor-trainer/src/data.rs:566-589)."""
import json

from ferrotensor_amd.data import MetricsWriter, TrainingExample


def test_next_token_example():
    e = TrainingExample.from_next_token([1, 2, 3, 4])
    assert (e.input_ids, e.target_ids, e.loss_mask) == ([1, 2, 3], [2, 3, 4], [1, 1, 1])
    short = TrainingExample.from_next_token([7])
    assert (short.input_ids, short.target_ids, short.loss_mask) == ([7], [7], [1])
    assert TrainingExample.from_next_token([]).as_tuple() == ([], [], [])


def test_sft_example_masks_only_response_tokens():
    e = TrainingExample.from_sft_prompt_response([10, 11, 12], [20, 21])
    assert e.input_ids == [10, 11, 12, 20]
    assert e.target_ids == [11, 12, 20, 21]
    assert e.loss_mask == [0, 0, 1, 1]
    # no prompt, or no response: every target is supervised
    assert TrainingExample.from_sft_prompt_response([], [1, 2, 3]).loss_mask == [1, 1]
    assert TrainingExample.from_sft_prompt_response([1, 2, 3], []).loss_mask == [1, 1]
    # one prompt token: the first target already is a response token
    assert TrainingExample.from_sft_prompt_response([5], [6, 7]).loss_mask == [1, 1]
    assert TrainingExample.from_sft_prompt_response([5], []).as_tuple() == ([5], [5], [1])


def test_metrics_log_lines(tmp_path):
    path = tmp_path / "metrics.jsonl"
    w = MetricsWriter(str(path))
    w.add_sequence(2.0, 10)
    w.add_sequence(4.0, 30)
    rec = w.log(3, 0.5, 2e-4)
    w.add_sequence(1.0, 5)
    w.log(4, 0.25, 1e-4)
    w.close()
    lines = [json.loads(l) for l in open(path)]
    assert [l["step"] for l in lines] == [3, 4]
    assert set(lines[0]) == {"step", "loss", "grad_norm", "lr", "tokens", "seconds", "elapsed"}
    assert lines[0]["loss"] == 3.5 and lines[0]["tokens"] == 40 and lines[1]["loss"] == 1.0 and lines[1]["tokens"] == 5
    assert rec["elapsed"] >= rec["seconds"] >= 0.0
