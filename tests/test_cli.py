"""The command line's own behaviour, without a GPU: exit codes as the reference's (0 for --help, 2 for a bad command
line, include/inferx/support/options.h:17-22), options from a --config file, the reference's option names."""
import pytest

from inferx_amd.engine import cli


def parse(argv):
    ap = cli.build_parser()
    first, _ = ap.parse_known_args(argv)
    if first.config:
        ap.set_defaults(**cli._config_file_defaults(ap, first.config))
    return ap.parse_args(argv)


def test_help_is_0_and_a_bad_command_line_is_2(capsys):
    with pytest.raises(SystemExit) as e:
        cli.main(["--help"])
    assert e.value.code == 0
    text = capsys.readouterr().out
    for option in ("--model", "--dtype", "--max-num-seqs", "--max-model-len", "--max-num-batched-tokens", "--block-size",
                   "--num-gpu-blocks-override", "--kv-cache-memory-bytes", "--gpu-memory-utilization", "--enforce-eager",
                   "--device", "--config", "--log-level", "--log-json", "--log-file", "--dump-logits"):
        assert option in text, option
    for bad in (["--no-such-flag"], ["--model", "x"], ["--model", "x", "--random-config", "y", "--prompt-ids", "1"],
                ["--model", "x", "--prompt-ids", "1", "--max-tokens", "0"], ["--model", "x", "--prompt-ids", "a,b"],
                ["--model", "x", "--prompt-ids", "1", "--dtype", "float16"]):
        with pytest.raises(SystemExit) as e:
            cli.main(bad)
        assert e.value.code == 2, bad


def test_options_from_a_config_file(tmp_path):
    toml = tmp_path / "options.toml"
    toml.write_text('max-model-len = 64\nmax_tokens = 3\ndtype = "fp32"\nenforce-eager = true\n'
                    'prompt-ids = ["1,2,3"]\ngpu-memory-utilization = 0.5\n')
    a = parse(["--config", str(toml), "--model", "m"])
    assert (a.max_model_len, a.max_tokens, a.dtype, a.enforce_eager, a.prompt_ids, a.gpu_memory_utilization) == \
        (64, 3, "fp32", True, ["1,2,3"], 0.5)
    assert parse(["--config", str(toml), "--model", "m", "--max-tokens", "9"]).max_tokens == 9  # the command line wins
    ini = tmp_path / "options.ini"
    ini.write_text("block-size = 32\nlog-level = info\nenforce-eager = no\n")
    a = parse(["--config", str(ini), "--model", "m"])
    assert (a.block_size, a.log_level, a.enforce_eager) == (32, "info", False)
    for text, needle in (("no-such-option = 1\n", "unknown option"), ('block-size = "wide"\n', "is not int"),
                         ('log-level = "loud"\n', "must be one of")):
        bad = tmp_path / "bad.toml"
        bad.write_text(text)
        with pytest.raises(SystemExit) as e:
            parse(["--config", str(bad), "--model", "m"])
        assert e.value.code == 2


def test_aliases_of_the_reference_s_options():
    a = parse(["m", "--num-blocks", "7", "--dtype", "bf16"])
    assert a.model_tag == "m" and a.num_gpu_blocks_override == 7 and a.dtype == "bf16"
