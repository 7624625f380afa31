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
