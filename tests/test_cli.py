"""Command-line parsing in the reference's manner (src/main.rs:147-296 of yusiwen/minfer):
defaults, option names, usage plus status 1 on a bad flag or value; and bench.py's refusal
of more than one GPU."""
import os
import subprocess
import sys

import pytest

from minfer_amd.cli import UsageError, main, parse_args, parse_prompts

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_defaults_are_the_references():
    o = parse_args(["model_dir", "--prompt-tokens", "1,2,3"])
    assert (o["temp"], o["top_k"], o["top_p"], o["repeat_penalty"]) == (0.8, 40, 0.95, 1.1)   # src/main.rs:55-69
    assert (o["frequency_penalty"], o["presence_penalty"], o["seed"], o["n_predict"], o["n_ctx"]) == (0.0, 0.0, 42, 512, 4096)
    assert o["model"] == "model_dir" and o["dtype"] == "bfloat16" and o["graph"] is True


def test_option_names_and_aliases():
    o = parse_args(["m", "--prompt-tokens", "1", "--greedy", "-n", "7", "--top-k", "0", "--top-p", "0.5",
                    "--repeat-penalty", "1.0", "--frequency-penalty", "0.2", "--presence-penalty", "0.3",
                    "--seed", "9", "--n-ctx", "128", "--n-slots", "3", "--stop-token", "5", "--stop-token", "6",
                    "--dtype", "float32", "--no-graph"])
    assert o["temp"] == 0.0 and o["n_predict"] == 7 and o["top_k"] == 0 and o["top_p"] == 0.5
    assert o["stop_tokens"] == [5, 6] and o["n_slots"] == 3 and o["dtype"] == "float32" and o["graph"] is False
    assert parse_args(["m", "--max-new", "3"])["n_predict"] == 3 and parse_args(["m", "--n-predict", "4"])["n_predict"] == 4
    assert parse_args(["m", "-t", "0.3"])["temp"] == 0.3
    r = parse_args(["--config", "c.json", "--random-weights", "--weight-seed", "5"])
    assert r["model"] is None and r["random_weights"] and r["config"] == "c.json" and r["weight_seed"] == 5


@pytest.mark.parametrize("argv,needle", [
    (["m", "--bogus"], "unknown option --bogus"),
    (["m", "--temp"], "--temp requires a value"),
    (["m", "--top-k", "many"], "cannot parse 'many'"),
    (["m", "extra"], "unexpected argument"),
])
def test_bad_arguments(argv, needle):
    with pytest.raises(UsageError, match=needle):
        parse_args(argv)


def test_usage_and_exit_status(capsys):
    assert main(["m", "--bogus"]) == 1
    err = capsys.readouterr().err
    assert "Error: unknown option --bogus" in err and "USAGE:" in err and "--prompt-tokens" in err
    assert main(["m"]) == 1 and "--prompt-tokens is required" in capsys.readouterr().err
    assert main(["--prompt-tokens", "1"]) == 1 and "model folder is required" in capsys.readouterr().err
    assert main(["m", "--prompt-tokens", "1", "--dtype", "int8"]) == 1
    assert main(["--help"]) == 0 and "USAGE:" in capsys.readouterr().err
    assert main(["-V"]) == 0 and "minfer_amd" in capsys.readouterr().out


def test_prompt_token_lists(tmp_path):
    assert parse_prompts("1,2,3") == [[1, 2, 3]]
    assert parse_prompts("1,2;3 4 ; 5") == [[1, 2], [3, 4], [5]]
    f = tmp_path / "p.txt"
    f.write_text("7,8\n\n9\n")
    assert parse_prompts("@" + str(f)) == [[7, 8], [9]]
    for bad in ("", ";", "1,x"):
        with pytest.raises(UsageError):
            parse_prompts(bad)


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2 and len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout
