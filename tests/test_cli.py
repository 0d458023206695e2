"""The command line (flow_engine/cli.py:48-118): doctor, inspect, random-weights and replay need no GPU;
generate runs on the GPU and leaves a JSONL log that replay prints."""
import json

import pytest
import torch

import plain_model as plain
from tiny_configs import TINY, make_folder
from tessweave_engine_amd import cli


def run(capsys, *argv):
    assert cli.main(list(argv)) == 0
    return capsys.readouterr().out


def test_doctor_inspect_random_weights_and_replay(tmp_path, capsys):
    report = json.loads(run(capsys, "doctor"))
    assert {"python", "platform", "torch", "gpu", "kernel_library"} <= set(report)
    cfg, page, _ = TINY["B"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    out = run(capsys, "random-weights", str(tmp_path / "config.json"), str(tmp_path / "model"), "--seed", "4").strip()
    assert out == str(tmp_path / "model")
    config, weights = plain.read_folder(tmp_path / "model")
    assert weights["model.layers.2.mlp.down_proj.weight"].shape == (cfg["hidden_size"], cfg["intermediate_size"])
    # the same seed gives the same bytes, another seed other ones
    run(capsys, "random-weights", str(tmp_path), str(tmp_path / "again"), "--seed", "4")
    run(capsys, "random-weights", str(tmp_path), str(tmp_path / "other"), "--seed", "5")
    again, other = plain.read_folder(tmp_path / "again")[1], plain.read_folder(tmp_path / "other")[1]
    assert all(torch.equal(weights[k], again[k]) for k in weights)
    assert not torch.equal(weights["lm_head.weight"], other["lm_head.weight"])
    # inspect: no weights are read (the folder holds only config.json); the byte formula of the reference
    info = json.loads(run(capsys, "inspect", str(tmp_path), "--kv-blocks", "10", "--block-size", "8"))
    per_token = 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"]
    assert info["kv_bf16_bytes"] == per_token * 2 * 80 and info["kv_fp32_bytes"] == per_token * 4 * 80
    assert info["architecture"]["num_hidden_layers"] == 3 and info["cache_groups"][0]["window"] is None
    assert "kv_bf16_bytes_by_formula" not in info               # head size 32: the device holds what the formula says
    # a head of 18 elements lies in 32 on the device: both figures are printed
    odd = tmp_path / "odd"
    odd.mkdir()
    (odd / "config.json").write_text(json.dumps(dict(cfg, head_dim=18, hidden_size=6 * 18)))
    info = json.loads(run(capsys, "inspect", str(odd), "--kv-blocks", "10", "--block-size", "8"))
    layers_heads = 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"]
    assert info["kv_bf16_bytes"] == layers_heads * 32 * 2 * 80 and info["kv_bf16_bytes_by_formula"] == layers_heads * 18 * 2 * 80
    assert info["kv_fp32_bytes_by_formula"] * 32 == info["kv_fp32_bytes"] * 18
    with pytest.raises(SystemExit):
        cli.main(["inspect", str(tmp_path), "--kv-blocks", "0"])
    capsys.readouterr()
    # replay prints the scheduler's events of a log and nothing else
    log = tmp_path / "run.jsonl"
    events = [{"event": "launch", "argv": ["x"]}, {"event": "admit", "request_id": "r1"},
              {"event": "step", "batch": 2}, {"event": "loaded"}, {"event": "first_token", "ttft_ms": 1.5},
              {"event": "finish", "reason": "length"}, {"event": "fatal", "error": "boom"}]
    log.write_text("".join(json.dumps(e) + "\n" for e in events) + "\n")
    shown = [json.loads(line) for line in run(capsys, "replay", str(log)).splitlines()]
    assert [e["event"] for e in shown] == ["admit", "step", "first_token", "finish", "fatal"]


def test_prompts_are_taken_out_of_a_command_line():
    argv = ["flow-inference", "generate", "m", "--prompt", "tell me", "--max-tokens", "3", "--prompt-ids=1,2,3",
            "--prompt-ids", "4,5", "--prompt=x y", "--prompt-file", "ids.txt", "--prompt"]
    assert cli.without_prompts(argv) == ["flow-inference", "generate", "m", "--prompt", "[REDACTED]", "--max-tokens", "3",
                                         "--prompt-ids=[REDACTED]", "--prompt-ids", "[REDACTED]", "--prompt=[REDACTED]",
                                         "--prompt-file", "ids.txt", "--prompt"]


@pytest.mark.gpu
def test_generate_prints_the_tokens_and_logs_the_run(tmp_path, capsys, device):
    make_folder(tmp_path / "model", "A")
    config, weights = plain.read_folder(tmp_path / "model")
    prompt = [5, 17, 3, 200, 41, 7, 99]
    want = plain.greedy(config, weights, prompt, 5)
    log = tmp_path / "logs" / "engine.jsonl"
    ids_file = tmp_path / "prompt.txt"
    ids_file.write_text(" ".join(str(t) for t in prompt))
    for source in (["--prompt-ids", ",".join(str(t) for t in prompt)], ["--prompt-file", str(ids_file)]):
        assert cli.main(["generate", str(tmp_path / "model"), *source, "--max-tokens", "5", "--dtype", "float32",
                         "--ignore-eos", "--prefill-chunk", "4", "--kv-blocks", "8", "--max-context", "64",
                         "--log", str(log)]) == 0
        captured = capsys.readouterr()
        assert [int(t) for t in captured.out.split()] == want
        usage = json.loads(captured.err.strip().splitlines()[-1])
        assert usage["type"] == "done" and usage["error"] is None
    kinds = [json.loads(line)["event"] for line in log.read_text().splitlines()]
    assert kinds[:2] == ["launch", "loaded"] and {"admit", "step", "first_token", "finish"} <= set(kinds)
    launches = [json.loads(line) for line in log.read_text().splitlines() if json.loads(line)["event"] == "launch"]
    shown = launches[0]["argv"]                                      # the command line given to main(), prompt removed
    assert shown[shown.index("--prompt-ids") + 1] == "[REDACTED]" and shown[:3] == ["flow-inference", "generate", str(tmp_path / "model")]
    assert ",".join(str(t) for t in prompt) not in log.read_text()
    shown = [json.loads(line)["event"] for line in run(capsys, "replay", str(log)).splitlines()]
    assert shown and set(shown) <= {"step", "admit", "finish", "first_token", "fatal"}
    with pytest.raises(SystemExit):
        cli.main(["generate", str(tmp_path / "model"), "--max-tokens", "2", "--max-context", "64", "--log", str(log)])    # no prompt given
    with pytest.raises(ValueError, match="max_position_embeddings"):
        cli.main(["generate", str(tmp_path / "model"), "--prompt-ids", "1", "--max-context", "4096", "--log", str(log)])
