"""The command line: subcommands, exit codes, and where output goes (bins/vipera/src/main.rs:66-100,
crates/vipera-errors/src/lib.rs:94-104: 0 ok, 1 usage, 2 bad input, 3 infeasible, 4 internal)."""
import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import CONFIG_A, CONFIG_B, make_folder, random_tokens

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
VIPERA = [sys.executable, os.path.join(ROOT, "bin", "vipera")]


class _Result:
    def __init__(self, returncode, stdout, stderr):
        self.returncode, self.stdout, self.stderr = returncode, stdout, stderr


def run(*args, binary=False):
    """Run the command line: in this process (fast), or the installed script when ``binary`` is set."""
    if binary:
        return subprocess.run(VIPERA + list(args), capture_output=True, text=True, timeout=300)
    import contextlib
    import io

    import vipera_rs_amd  # noqa: F401
    from vipera_rs_amd.cli import main
    out, err = io.StringIO(), io.StringIO()
    with contextlib.redirect_stdout(out), contextlib.redirect_stderr(err):
        code = main(list(args))
    return _Result(code, out.getvalue(), err.getvalue())


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return make_folder(tmp_path_factory.mktemp("cli_model"), CONFIG_A, 0, torch.float32)


def test_help_and_usage_errors():
    ok = run("--help", binary=True)
    assert ok.returncode == 0 and "generate" in ok.stdout and "EXIT CODES" in ok.stdout
    none = run()
    assert none.returncode == 1 and "USAGE" in none.stderr and none.stdout == ""
    bad = run("frobnicate", binary=True)
    assert bad.returncode == 1 and bad.stderr.strip() == 'vipera: unknown command "frobnicate"' and bad.stdout == ""


def test_model_info_reads_headers_only(folder):
    out = run("model-info", folder, "--json")
    assert out.returncode == 0, out.stderr
    info = json.loads(out.stdout)
    assert info["architecture"] == "Qwen2ForCausalLM" and info["parameter_count"] == 90688
    assert info["tensor_count"] == 26 and info["layer_count"] == 2 and info["vocab_size"] == 256
    assert info["tied"] is True and info["tensor_types"] == {"F32": 26} and len(info["identity"]) == 16
    text = run("model-info", folder)
    assert text.returncode == 0 and "parameter_count: 90688" in text.stdout
    flag = run("model-info", folder, "--verbose")
    assert flag.returncode == 1 and 'unknown flag "--verbose"' in flag.stderr
    missing = run("model-info", os.path.join(folder, "nope"))
    assert missing.returncode == 2 and missing.stderr.startswith("vipera: ")
    assert run("model-info").returncode == 1


def test_plan_predicts_memory_and_refuses_what_does_not_fit(folder, tmp_path):
    out = run("plan", folder, "--ctx", "256", "--batch", "4", "--dtype", "float32", "--json")
    assert out.returncode == 0, out.stderr
    plan = json.loads(out.stdout)
    # keys and values cost 2 * kv_heads * head_dim * bytes per position and layer (planner.rs:191-206)
    assert plan["kv_bytes_per_token"] == 2 * 2 * 16 * 4 * 2
    assert plan["kv_blocks"] == 4 * 16 and plan["kv_bytes"] == 4 * 256 * plan["kv_bytes_per_token"]
    assert plan["feasible"] is True and plan["violations"] == []
    assert plan["weight_bytes"] == 90688 * 4
    too_long = run("plan", folder, "--ctx", "100000")
    assert too_long.returncode == 2 and "exceeds the model's maximum" in too_long.stderr
    # a model whose cache cannot fit the device: exit 3 with the violation spelled out
    big = dict(CONFIG_B, num_hidden_layers=200, num_key_value_heads=3, max_position_embeddings=4_000_000)
    cfg_path = tmp_path / "big.json"
    cfg_path.write_text(json.dumps(big))
    from vipera_rs_amd.config import config_from_dict
    config_from_dict(big).save(str(tmp_path / "bigmodel"))
    open(tmp_path / "bigmodel" / "model.safetensors", "wb").write((8).to_bytes(8, "little") + b"{}      ")
    no_fit = run("plan", str(tmp_path / "bigmodel"), "--ctx", "4000000", "--batch", "64", "--json")
    assert no_fit.returncode == 3, no_fit.stderr
    violation = json.loads(no_fit.stdout)["violations"][0]
    assert violation["constraint"] == "device_memory" and violation["required_bytes"] > violation["available_bytes"]


def test_plan_counts_the_weights_as_the_loader_keeps_them(tmp_path):
    """Whatever floating-point type a folder stores, the plan's ``weight_bytes`` is the sum over the tensors of the
    size in the dtype the loader keeps each in (planner.rs:266-430 predicts what the backend then allocates)."""
    import vipera_rs_amd  # noqa: F401
    from vipera_rs_amd.cli import plan_model
    from vipera_rs_amd.config import config_from_dict
    from vipera_rs_amd.models import declare_model
    from vipera_rs_amd.weights import Checkpoint, kept_dtype, write_safetensors
    specs = {s.name: s for s in declare_model(config_from_dict(CONFIG_B))}
    source = make_folder(tmp_path / "f32", CONFIG_B, 1, torch.float32)
    ck = Checkpoint(source)
    tensors = {name: ck.read(name).clone() for name in ck.names()}
    ck.close()
    matrices = sum(t.numel() for n, t in tensors.items() if specs[n].role == "matrix")
    vectors = sum(t.numel() for n, t in tensors.items() if specs[n].role == "vector")
    assert matrices > 0 and vectors > 0
    for stored in (torch.float32, torch.bfloat16, torch.float16):
        folder = str(tmp_path / str(stored).split(".")[-1])
        config_from_dict(CONFIG_B).save(folder)
        write_safetensors(os.path.join(folder, "model.safetensors"), ((n, t.to(stored)) for n, t in tensors.items()))
        for run_as, keep in (("bfloat16", False), ("bfloat16", True), ("float32", False)):
            run_dtype = torch.float32 if run_as == "float32" else torch.bfloat16
            want = sum(t.numel() * torch.empty(0, dtype=kept_dtype(specs[n], stored, run_dtype, keep)).element_size()
                       for n, t in tensors.items())
            plan = plan_model(folder, 64, 1, run_as, 16, keep_float32=keep)
            assert plan["weight_bytes"] == want, (stored, run_as, keep)
            kept32 = run_as == "float32" or (keep and stored == torch.float32)
            assert want == matrices * (4 if kept32 else 2) + vectors * 4
    # the command line says the same
    out = run("plan", str(tmp_path / "float32"), "--ctx", "64", "--json")
    assert json.loads(out.stdout)["weight_bytes"] == matrices * 2 + vectors * 4
    out = run("plan", str(tmp_path / "float32"), "--ctx", "64", "--keep-float32", "--json")
    assert json.loads(out.stdout)["weight_bytes"] == matrices * 4 + vectors * 4


def test_a_shape_no_kernel_takes_is_refused_when_the_model_is_opened(tmp_path):
    """A head width above the attention kernels' limit: `unsupported` (exit 2) from every subcommand that opens the
    model, before any weight is read (the reference refuses while it reads the header, model.rs:1323-1328,
    1367-1383; exit codes errors/lib.rs:94-104), not an internal error from the first step."""
    wide = dict(CONFIG_B, hidden_size=64, num_attention_heads=1, num_key_value_heads=1, head_dim=272,
                intermediate_size=32, vocab_size=40, num_hidden_layers=1)
    folder = make_folder(tmp_path / "wide", wide, 1)
    for command in (["model-info", folder], ["plan", folder], ["generate", folder, "--prompt-ids", "1 2 3"]):
        out = run(*command)
        assert out.returncode == 2, (command, out.stderr)
        assert out.stderr.startswith("vipera: ") and "head_dim 272" in out.stderr and "limit of 256" in out.stderr
        assert out.stdout == ""
    # the weights are not looked at: the same refusal without them
    os.remove(os.path.join(folder, "model.safetensors"))
    assert "head_dim 272" in run("plan", folder).stderr


def test_random_model_writes_a_loadable_folder(tmp_path):
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(CONFIG_B))
    out = run("random-model", str(cfg_path), str(tmp_path / "m"), "--seed", "5", "--dtype", "bfloat16")
    assert out.returncode == 0, out.stderr
    info = json.loads(run("model-info", str(tmp_path / "m"), "--json").stdout)
    assert info["dtype"] == "BF16" and info["tied"] is False and info["head_dim"] == 32
    assert run("random-model", str(cfg_path)).returncode == 1
    bad = tmp_path / "bad.json"
    bad.write_text(json.dumps(dict(CONFIG_B, hidden_act="relu")))
    refused = run("random-model", str(bad), str(tmp_path / "m2"))
    assert refused.returncode == 2 and "hidden_act" in refused.stderr


def test_generate_checks_its_arguments_before_loading(folder):
    assert run("generate", folder).returncode == 1
    assert run("generate", "--prompt-ids", "1 2").returncode == 1
    zero = run("generate", folder, "--prompt-ids", "1 2", "--max-tokens", "0")
    assert zero.returncode == 2 and "--max-tokens must be at least 1" in zero.stderr
    hot = run("generate", folder, "--prompt-ids", "1 2", "--temperature", "-1")
    assert hot.returncode == 2 and "temperature" in hot.stderr
    nan = run("generate", folder, "--prompt-ids", "1 x 2")
    assert nan.returncode == 2


@pytest.mark.gpu
def test_generate_prints_token_ids_and_json(folder):
    from plain import qwen2_plain
    cfg, weights = qwen2_plain.load_folder(folder)
    prompt = random_tokens(256, 9, 77)
    want = qwen2_plain.greedy_generate(cfg, weights, prompt, 6)
    ids = " ".join(str(t) for t in prompt)
    text = run("generate", folder, "--prompt-ids", ids, "--max-tokens", "6", "--dtype", "float32", binary=True)
    assert text.returncode == 0, text.stderr
    assert [int(t) for t in text.stdout.split()] == want
    out = run("generate", folder, "--prompt-ids", ids, "--max-tokens", "6", "--dtype", "float32", "--json")
    report = json.loads(out.stdout)
    assert report["tokens"] == want and report["prompt_tokens"] == 9 and report["generated_tokens"] == 6
    assert report["finish"] == "length" and report["processed_tokens"] == 9 + 5 and set(report["micros"]) == {"schedule", "allocate", "compute", "sample"}
    seeded = [run("generate", folder, "--prompt-ids", ids, "--max-tokens", "8", "--temperature", "0.9", "--seed", "4",
                  "--dtype", "float32").stdout for _ in range(2)]
    assert seeded[0] == seeded[1] and len(seeded[0].split()) == 8
    long = run("generate", folder, "--prompt-ids", ids, "--ctx", "100000")
    assert long.returncode == 2 and "exceeds the model's maximum" in long.stderr
    outside = run("generate", folder, "--prompt-ids", "1 999", "--dtype", "float32")
    assert outside.returncode == 2 and "outside the vocabulary" in outside.stderr


@pytest.mark.gpu
def test_sample_subcommand():
    out = run("sample", "--logits", "0.1,2.5,2.5,-1", "--temperature", "0", "--json")
    assert out.returncode == 0, out.stderr
    assert json.loads(out.stdout)["tokens"] == [1]
    many = run("sample", "--logits", "1.0986123,0", "--temperature", "1", "--top-k", "0", "--top-p", "1", "--min-p", "0",
               "--count", "400", "--seed", "3")
    draws = [int(t) for t in many.stdout.split()]
    assert len(draws) == 400 and abs(draws.count(0) / 400 - 0.75) < 0.08
    assert run("sample").returncode == 1
    assert run("sample", "--logits", "nan,nan").returncode == 2
