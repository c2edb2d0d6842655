"""The command line's reading of its options (no GPU), after
src/main.rs:179-345 of the reference."""
import pytest

from torchless_rs_amd.cli import main, parse_args, parse_ids
from torchless_rs_amd.sampling import SamplingConfig


def test_defaults_and_values():
    o, pos = parse_args(["model_dir", "1 2 3"])
    assert o["--temperature"] == 0.7 and o["--max-tokens"] is None and o["--seed"] == 0   # main.rs:165
    assert pos == ["model_dir", "1 2 3"]
    o, pos = parse_args(["--temperature", "0", "--top-k", "40", "--top-p", "0.9", "--max-tokens", "5",
                         "--max-seq-len", "128", "--seed", "4", "--dtype", "float32", "--debug", "m"])
    assert (o["--temperature"], o["--top-k"], o["--top-p"], o["--max-tokens"], o["--max-seq-len"],
            o["--seed"], o["--dtype"], o["--debug"]) == (0.0, 40, 0.9, 5, 128, 4, "float32", True)


@pytest.mark.parametrize("argv, text", [
    (["--bogus", "m"], "unknown option '--bogus'"),                      # main.rs:335-339
    (["m", "--max-tokens"], "--max-tokens requires a value"),            # main.rs:262-266
    (["--temperature", "hot", "m"], "invalid --temperature value 'hot'"),
    (["--top-k", "1.5", "m"], "invalid --top-k value"),
])
def test_errors_exit_1(argv, text, capsys):
    with pytest.raises(SystemExit) as e:
        parse_args(argv)
    assert e.value.code == 1 and text in capsys.readouterr().err


def test_help_and_usage(capsys):
    with pytest.raises(SystemExit) as e:
        parse_args(["--help"])
    assert e.value.code == 0 and "--max-tokens" in capsys.readouterr().err
    assert main([]) == 1
    assert main(["m"]) == 1 and "no prompt" in capsys.readouterr().err
    assert main(["--random-weights", "m"]) == 1
    assert main(["m", "one two"]) == 1


def test_a_failed_run_is_an_error_line_and_exit_1(tmp_path, capsys):
    """What `generate` raises (here: a folder that holds no model, or no GPU) comes out as the
    other errors do, not as a traceback."""
    assert main([str(tmp_path / "no_such_model"), "1 2 3"]) == 1
    err = capsys.readouterr().err
    assert err.startswith("Error: ") and "Traceback" not in err


def test_default_number_of_new_tokens_follows_the_context():
    """src/main.rs:140-153: a quarter of the context, clamped to 1024 (2048 from 4096 on) .. 32768."""
    from torchless_rs_amd.api import default_max_tokens
    assert default_max_tokens(2048) == 1024 and default_max_tokens(4095) == 1024
    assert default_max_tokens(4096) == 2048 and default_max_tokens(32768) == 8192
    assert default_max_tokens(1 << 20) == 32768


def test_ids_and_sampling_names():
    assert parse_ids("1, 5 17") == [1, 5, 17]
    assert SamplingConfig().temperature == 1.0                            # sampler/mod.rs:46-54
    assert SamplingConfig.greedy().is_greedy and not SamplingConfig.with_temperature(0.8).is_greedy


def test_bench_serves_one_gpu_only():
    import os
    import subprocess
    import sys
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(repo, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout
