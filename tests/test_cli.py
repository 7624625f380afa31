"""The command line's handling of its own arguments (no GPU): usage errors exit with status 2 and say what is wrong
(the reference's flag discipline: /root/reference/src/cli/main.cpp:100-284)."""

import json

import pytest

from llmx_amd import cli


def run(argv, capsys):
    try:
        rc = cli.main(argv)
    except SystemExit as e:       # argparse's own exit on a usage error
        rc = e.code
    out = capsys.readouterr()
    return rc, out.out, out.err


def test_a_flag_given_twice_is_refused(capsys):
    rc, _, err = run(["generate", "m", "1,2", "--temp", "0", "--temp", "1"], capsys)
    assert rc == 2 and "given twice" in err
    rc, _, err = run(["generate", "m", "1,2", "-n", "3", "--max-tokens", "4"], capsys)
    assert rc == 2 and "given twice" in err


def test_unknown_flags_and_commands_are_usage_errors(capsys):
    assert run(["generate", "m", "1,2", "--no-such-flag"], capsys)[0] == 2
    assert run(["serve"], capsys)[0] == 2
    assert run([], capsys)[0] == 2


def test_bench_passes_its_flags_on(capsys):
    rc, out, _ = run(["bench", "--gpus", "2"], capsys)
    assert rc == 2 and "one GPU" in out


def test_replay_has_its_own_parser(capsys):
    rc, _, err = run(["replay", "--model", "m", "--dtype", "float16", "--out", "o", "--max-tokens", "64"], capsys)
    assert rc == 2 and "--dtype" in err


def test_prompts_are_token_ids(tmp_path, capsys):
    cfg = {"architectures": ["MiniMaxM3ForCausalLM"]}
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    rc, _, err = run(["perplexity", str(tmp_path), "7"], capsys)
    assert rc == 2 and "at least 2" in err
    rc, _, err = run(["logits", str(tmp_path), "five six"], capsys)
    assert rc == 2 and "token ids" in err
    rc, _, err = run(["logits", str(tmp_path)], capsys)
    assert rc == 2 and "needs token ids" in err


def test_sampling_ranges_are_checked_before_anything_is_loaded(tmp_path, capsys):
    rc, _, err = run(["generate", str(tmp_path), "1,2", "--topp", "1.5"], capsys)
    assert rc in (1, 2) and "top_p" in err
    rc, _, err = run(["generate", str(tmp_path), "1,2", "--stop", "x"], capsys)
    assert rc == 2 and "token ids" in err


def test_config_and_random_name_a_model_without_a_folder(tmp_path, capsys):
    """`--config JSON --random SEED` stands in the model folder's place; the two go together and leave the prompt as
    the only positional (the run itself needs the GPU and is tested there)."""
    rc, _, err = run(["generate", "--config", "c.json", "1,2"], capsys)
    assert rc == 2 and "--config and --random go together" in err
    rc, _, err = run(["generate", "--random", "3", "m", "1,2"], capsys)
    assert rc == 2 and "--config and --random go together" in err
    rc, _, err = run(["generate"], capsys)
    assert rc == 2 and "needs a model folder, or --config JSON --random SEED" in err
    rc, _, err = run(["generate", "--config", str(tmp_path / "none.json"), "--random", "0", "1,2"], capsys)
    assert rc == 2 and "none.json" in err
    rc, _, err = run(["generate", "--config", "c.json", "--random", "0", "1,2", "extra"], capsys)
    assert rc == 2 and "unexpected argument 'extra'" in err
    bad = tmp_path / "c.json"
    bad.write_text(json.dumps({"architectures": ["MiniMaxM3ForCausalLM"], "head_dim": 16}))
    rc, _, err = run(["generate", "--config", str(bad), "--random", "0", "1,2"], capsys)
    assert rc == 1 and "missing key" in err


def test_cache_types_and_device_are_the_reference_flags_with_this_engines_limits(tmp_path, capsys):
    """`--cache-type-k/-ctk`, `--cache-type-v/-ctv` and `--device` exist as in the reference
    (/root/reference/src/cli/main.cpp:120,544-555); the cache has the activations' type and the device is a GPU, and
    anything else is a usage error before a model is read."""
    rc, _, err = run(["generate", str(tmp_path), "1,2", "-ctk", "f32"], capsys)
    assert rc == 2 and "--cache-type-k f32" in err and "--dtype bf16" in err
    rc, _, err = run(["generate", str(tmp_path), "1,2", "--dtype", "f32", "--cache-type-v", "f16"], capsys)
    assert rc == 2 and "--cache-type-v f16" in err
    rc, _, err = run(["logits", str(tmp_path), "1,2", "--device", "cpu"], capsys)
    assert rc == 2 and "runs on a GPU only" in err
    # the matching type passes these checks (and then fails on the empty folder, not on usage)
    rc, _, err = run(["generate", str(tmp_path), "1,2", "--dtype", "f32", "-ctk", "f32", "-ctv", "f32", "--device", "cuda:0"], capsys)
    assert rc == 1 and "cache-type" not in err


def test_bench_with_a_model_is_the_reference_bench(capsys):
    """`bench --model` is parsed here (the reference's --p --n --r --seqs --depth, main.cpp:67-75); without a model
    the flags go on to bench.py."""
    rc, _, err = run(["bench", "--model", "m", "--p", "0"], capsys)
    assert rc == 2 and "--p must be at least 1" in err
    rc, _, err = run(["bench", "--model", "m", "--seqs", "2", "--depth", "8"], capsys)
    assert rc == 2 and "goes with one sequence" in err
    rc, _, err = run(["bench", "--model", "m", "--p", "4", "--p", "5"], capsys)
    assert rc == 2 and "given twice" in err
    rc, _, err = run(["bench", "--config", "c.json", "--n", "3"], capsys)
    assert rc == 2 and "--config and --random go together" in err
