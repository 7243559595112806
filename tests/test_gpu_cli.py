"""The command line in-process on the GPU: generate, benchmark and inspect on tiny model
folders, against the plain implementation where tokens are decided."""

import json

import pytest

import plain_lfm2 as plain
from helpers import make_model, random_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_model(str(root / name), name, seed=33) for name in ("A", "B")}


def run(capsys, *argv):
    from flyweight_amd.cli import main
    status = main(list(argv))
    captured = capsys.readouterr()
    return status, captured.out, captured.err


@pytest.mark.parametrize("name", ["A", "B"])
def test_generate_prints_the_plain_models_greedy_tokens(folders, name, capsys, tmp_path):
    config, weights = plain.read_folder(folders[name])
    prompt = random_tokens(config["vocab_size"], 11, seed=4)
    expected = plain.greedy(config, weights, prompt, 6)
    ids = ",".join(str(t) for t in prompt)
    # the model's eos must not end the generation early
    common = ("--max-tokens", "6", "--temperature", "0", "--dtype", "float32", "--ignore-eos")
    status, out, _ = run(capsys, "generate", folders[name], "--tokens", ids, *common)
    assert status == 0 and [int(t) for t in out.split()] == expected
    # the same from a file, in turns of several decode steps; a stop token ends it behind that token
    listed = tmp_path / "prompt.txt"
    listed.write_text(" ".join(str(t) for t in prompt))
    status, out, _ = run(capsys, "generate", folders[name], "--tokens-file", str(listed), "--max-new-tokens", "6",
                         "--temperature", "0", "--dtype", "float32", "--decode-steps-per-turn", "4",
                         "--stop-token", str(expected[3]))
    assert status == 0 and [int(t) for t in out.split()] == expected[:expected.index(expected[3]) + 1]


def test_generate_with_a_seed_reproduces_and_refuses_what_it_cannot_do(folders, capsys):
    folder = folders["B"]
    sampled = ("generate", folder, "--tokens", "3,1,4,1,5", "--max-tokens", "12", "--temperature", "0.8", "--top-k", "40",
               "--seed", "7", "--ignore-eos")
    first = run(capsys, *sampled)
    second = run(capsys, *sampled)
    assert first[0] == 0 and first[1] == second[1] and len(first[1].split()) == 12
    status, out, err = run(capsys, "generate", folder, "--max-tokens", "3")
    assert status == 2 and "--tokens" in err and out == ""
    status, out, err = run(capsys, "generate", folder, "--tokens", "1,2", "--temperature", "-1")
    assert status == 1 and "temperature" in err
    status, out, err = run(capsys, "generate", folder, "--tokens", "1,2", "--stop-token", "100000")
    assert status == 1 and "stop token 100000 is outside the vocabulary" in err
    status, out, err = run(capsys, "generate", folder, "--tokens", "1,100000")
    assert status == 1 and "token id 100000 at place 1" in err
    # a cache of two pages holds 128 tokens of one request: a request that needs a third page is refused by name
    status, out, err = run(capsys, "generate", folder, "--tokens", "1,2", "--max-tokens", "100", "--num-pages", "2", "--temperature", "0",
                           "--ignore-eos")
    assert status == 0 and len(out.split()) == 100
    status, out, err = run(capsys, "generate", folder, "--tokens", "1,2", "--max-tokens", "200", "--num-pages", "2", "--ignore-eos")
    assert status == 1 and "cache pages" in err
    status, out, err = run(capsys, "generate", folder + "-missing", "--tokens", "1,2")
    assert status == 1 and err.startswith("flyweight-amd:")


def test_benchmark_and_inspect_print_json(folders, capsys):
    status, out, _ = run(capsys, "benchmark", folders["A"], "--tokens", "5,6,7", "--warmup", "2", "--iterations", "9")
    report = json.loads(out)
    assert status == 0 and report["prompt_tokens"] == 3 and report["iterations"] == 9
    assert report["decode_tokens_per_second"] > 0 and 0 < report["median_seconds"] <= report["p99_seconds"]
    assert report["prompt_and_first_token_seconds"] > 0 and report["prepare_seconds"] > 0
    assert report["decode_first_window_tokens_per_second"] > 0 and report["decode_last_window_tokens_per_second"] > 0
    assert report["generated_tokens"] == 1 + 2 + 9 and report["request_seconds"] > report["prompt_and_first_token_seconds"]
    # the same with the per-kernel profile: GPU time per kernel entry point, and steps without graphs
    from flyweight_amd.kernels import ops
    try:
        status, out, _ = run(capsys, "benchmark", folders["A"], "--tokens", "5,6,7", "--warmup", "1", "--iterations", "4", "--kernel-profile")
    finally:
        ops.kernel_profile(False)
    kernels = json.loads(out)["kernels"]
    assert status == 0 and kernels["fw_embed_rows"]["calls"] >= 6 and kernels["fw_gemm_decode"]["gpu_ms"] > 0
    assert all(entry["host_launch_ms"] > 0 and entry["max_us"] > 0 for entry in kernels.values())
    status, out, _ = run(capsys, "inspect", folders["B"])
    shown = json.loads(out)
    config, weights = plain.read_folder(folders["B"])
    assert status == 0 and shown["architecture"] == "Lfm2ForCausalLM"
    assert shown["config"]["hidden_size"] == config["hidden_size"] and shown["derived"]["layers"] == config["num_hidden_layers"]
    assert set(shown["tensors"]) == set(weights)
    assert shown["derived"]["parameters"] == sum(int(w.size) for w in weights.values())
