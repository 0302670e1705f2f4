"""The command line: ``generate``, ``model-info``, ``plan`` and ``sample``.

Subcommands, option names and their meanings, defaults and exit codes follow the reference's binary
(bins/vipera/src/main.rs:32-64 usage, 548-631 ``generate`` flags, 161-251 ``model-info`` and ``plan``,
1006-1122 ``sample``): flags are parsed by hand, an unknown flag is a usage error (exit 1), bad input
is exit 2, a plan that does not fit is exit 3, anything else exit 4; standard output carries only what
was asked for and errors go to standard error as ``vipera: <error>`` (main.rs:66-74).  What differs:
a model is a folder (``config.json`` + safetensors), and prompts are token ids, since tokenizing is
not part of this engine.
"""
from __future__ import annotations

import json
import os
import sys
import time
from typing import Dict, List, Optional

from .errors import InfeasibleError, InvalidArgumentError, UsageError, ViperaError

USAGE = """\
vipera: inference engine for one MI355X

USAGE:
    vipera model-info <model-dir> [--json]
    vipera plan <model-dir> [--ctx N] [--batch N] [--dtype bfloat16|float32] [--block-size N] [--keep-float32]
                [--json]
    vipera sample [--logits CSV | --logits-file PATH] [--count N] [--seed N] [--temperature F]
                  [--top-k N] [--top-p F] [--min-p F] [--repetition-penalty F] [--recent IDS] [--json]
    vipera generate <model-dir> (--prompt-ids IDS | --prompt-ids-file PATH) [--max-tokens N] [--ctx N]
                    [--dtype bfloat16|float32] [--block-size N] [--temperature F] [--top-k N] [--top-p F]
                    [--min-p F] [--repetition-penalty F] [--seed N] [--keep-float32] [--json]
    vipera random-model <config.json> <out-dir> [--seed N] [--dtype bfloat16|float32]
    vipera --help

COMMANDS:
    model-info    Print the model's architecture, sizes and tensor summary (reads headers only)
    plan          Predict device memory and per-step work for a context and batch without loading the model
    sample        Sample token ids from logits with a fixed seed and print the result
    generate      Run the model on the GPU and print the token ids it writes next
    random-model  Write a model folder with seeded random weights for a configuration

EXIT CODES:
    0 success, 1 usage, 2 bad input, 3 infeasible plan, 4 internal
"""

HBM_BYTES = 288 * 1000 ** 3
DEVICE_RESERVE = 16 * 1024 * 1024  # kept free on the device, as the reference's planner does (planner.rs:23)


class Args:
    """Hand-rolled flag parsing in the reference's manner (main.rs:562-631)."""

    def __init__(self, argv: List[str], command: str, flags: Dict[str, bool], positional: int):
        self.values: Dict[str, str] = {}
        self.switches = set()
        self.positional: List[str] = []
        index = 0
        while index < len(argv):
            arg = argv[index]
            if arg in flags:
                if flags[arg]:
                    if index + 1 >= len(argv):
                        raise UsageError(f"{arg} needs a value")
                    self.values[arg] = argv[index + 1]
                    index += 1
                else:
                    self.switches.add(arg)
            elif arg.startswith("-") and not _is_number(arg):
                raise UsageError(f"unknown flag \"{arg}\" for {command}")
            else:
                if len(self.positional) >= positional:
                    raise UsageError(f"unexpected extra argument \"{arg}\"")
                self.positional.append(arg)
            index += 1

    def number(self, flag: str, default, kind=float):
        if flag not in self.values:
            return default
        try:
            return kind(self.values[flag])
        except ValueError:
            raise InvalidArgumentError(f"{flag} expects a number, got \"{self.values[flag]}\"") from None


def _is_number(text: str) -> bool:
    try:
        float(text)
        return True
    except ValueError:
        return False


def _ids(text: str, what: str) -> List[int]:
    try:
        return [int(part) for part in text.replace(",", " ").split()]
    except ValueError:
        raise InvalidArgumentError(f"{what} expects token ids separated by spaces or commas") from None


def _sampling(args: Args, temperature_default: float):
    from .sampling import SamplingParams

    params = SamplingParams(
        temperature=args.number("--temperature", temperature_default),
        top_k=args.number("--top-k", 40, int),
        top_p=args.number("--top-p", 0.95),
        min_p=args.number("--min-p", 0.05),
        repetition_penalty=args.number("--repetition-penalty", 1.0),
        seed=args.number("--seed", 0, int),
    )
    params.validate()
    return params


def _emit(text: str) -> None:
    sys.stdout.write(text)
    sys.stdout.flush()


# --- model-info -----------------------------------------------------------------------------------
def model_summary(folder: str) -> dict:
    import torch

    from .config.registry import load_config
    from .models import check_model, declare_model
    from .weights import Checkpoint

    config = load_config(folder)
    check_model(config, torch.bfloat16)        # a model that no kernel takes is refused as one, not described
    checkpoint = Checkpoint(folder)
    try:
        dtypes: Dict[str, int] = {}
        parameters = 0
        identity = 0xCBF29CE484222325  # FNV-1a over names and shapes: a stable fingerprint of the layout
        for name in sorted(checkpoint.names()):
            info = checkpoint.info(name)
            count = 1
            for dim in info.shape:
                count *= dim
            parameters += count
            dtypes[info.dtype] = dtypes.get(info.dtype, 0) + 1
            for byte in f"{name}:{info.dtype}:{info.shape}".encode():
                identity = ((identity ^ byte) * 0x100000001B3) & ((1 << 64) - 1)
        checkpoint.check(declare_model(config))
        summary = {
            "architecture": config.architecture,
            "identity": f"{identity:016x}",
            "tensor_count": len(checkpoint.names()),
            "parameter_count": parameters,
            "dtype": max(dtypes, key=dtypes.get) if dtypes else None,
            "context_limit": config.context_limit,
            "layer_count": len(config.layer_specs()),
            "vocab_size": getattr(config, "vocab_size", None),
            "hidden": getattr(config, "hidden_size", None),
            "heads": getattr(config, "num_attention_heads", None),
            "kv_heads": getattr(config, "num_key_value_heads", None),
            "head_dim": getattr(config, "head_dim", None),
            "intermediate": getattr(config, "intermediate_size", None),
            "tied": getattr(config, "tie_word_embeddings", None),
            "tensor_types": dtypes,
        }
        return {key: value for key, value in summary.items() if value is not None}  # absent, not null
    finally:
        checkpoint.close()


def model_info_command(argv: List[str]) -> int:
    args = Args(argv, "model-info", {"--json": False}, 1)
    if not args.positional:
        raise UsageError("model-info needs a model folder")
    summary = model_summary(args.positional[0])
    if "--json" in args.switches:
        _emit(json.dumps(summary, indent=2) + "\n")
    else:
        for key, value in summary.items():
            _emit(f"{key}: {value}\n")
    return 0


# --- plan -------------------------------------------------------------------------------------------
def plan_model(folder: str, ctx: Optional[int], batch: int, dtype: str, block_size: int,
               keep_float32: bool = False) -> dict:
    """Bytes on the device and work per step, from the configuration and the tensor headers alone.

    The weights are counted in the dtypes the loader keeps them in (``weights.kept_bytes``: matrices in the run's
    dtype whatever the folder stores, or with ``keep_float32`` 32-bit ones as stored), so the plan predicts what
    loading then allocates, as the reference's planner does for its backend
    (crates/vipera-core/src/planner.rs:266-430).  The cache costs ``2 * kv_heads * head_dim * bytes`` per position
    and attention layer, the reference's arithmetic (planner.rs:191-206).
    """
    import torch

    from .cache import cache_bytes
    from .config.registry import load_config
    from .models import check_model, declare_cache_needs, declare_model
    from .weights.checkpoint import MATRIX, Checkpoint, kept_bytes, kept_dtype

    config = load_config(folder)
    if ctx is None:
        ctx = min(config.context_limit, 2048)
    if ctx > config.context_limit:
        from .errors import UnsupportedError
        raise UnsupportedError(f"requested context {ctx} exceeds the model's maximum of {config.context_limit}")
    if ctx < 1 or batch < 1 or block_size < 1:
        raise InvalidArgumentError("--ctx, --batch and --block-size must be at least 1")
    element = 4 if dtype == "float32" else 2
    run_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    specs = declare_model(config)
    check_model(config, run_dtype)             # what no kernel takes is refused before any byte is counted
    checkpoint = Checkpoint(folder)
    try:
        weight_bytes = kept_bytes(checkpoint, specs, run_dtype, keep_float32)
        matrix_elements = matrix_bytes = 0
        for spec in specs:
            present = spec.name in checkpoint.tensors
            if spec.role != MATRIX or (spec.optional and not present):
                continue
            count = 1
            for dim in spec.shape:
                count *= dim
            matrix_elements += count
            stored = checkpoint.info(spec.name).torch_dtype if present else run_dtype
            matrix_bytes += count * (4 if kept_dtype(spec, stored, run_dtype, keep_float32) == torch.float32 else 2)
        head_name = f"{config.head_spec().params['name']}.weight"
        tied = bool(config.head_spec().params.get("tied_to")) and head_name not in checkpoint.tensors
    finally:
        checkpoint.close()
    emb = config.embedding_spec().params
    embedding_elements = int(emb["vocab"]) * int(emb["width"])
    head_elements = embedding_elements
    kv_per_token, state_per_slot = cache_bytes(declare_cache_needs(config), element)
    blocks = batch * ((ctx + block_size - 1) // block_size)
    kv_bytes = blocks * block_size * kv_per_token
    state_bytes = (batch + 1) * state_per_slot      # one row per request and the scratch row of padding entries
    workspace = 2048 * (int(emb["width"]) * 4 + int(emb["vocab"]) * 4) + 256 * 1024 * 1024
    total = weight_bytes + kv_bytes + state_bytes + workspace + DEVICE_RESERVE
    # a decode step reads every matrix once (the embedding table only when it is also the head)
    step_weights = matrix_bytes * (matrix_elements - (0 if tied else embedding_elements)) // max(matrix_elements, 1)
    linear_elements = matrix_elements - embedding_elements - (0 if tied else head_elements)
    plan = {
        "dtype": dtype, "context": ctx, "batch": batch, "block_size": block_size,
        "weight_bytes": weight_bytes, "kv_bytes_per_token": kv_per_token, "kv_blocks": blocks,
        "kv_bytes": kv_bytes, "state_bytes": state_bytes, "workspace_bytes": workspace, "reserve_bytes": DEVICE_RESERVE,
        "required_bytes": total, "available_bytes": HBM_BYTES,
        "decode_step_read_bytes": step_weights + batch * (ctx * kv_per_token + state_per_slot),
        "prefill_flops_per_token_linear": 2 * linear_elements,
        "feasible": total <= HBM_BYTES, "violations": [],
    }
    if not plan["feasible"]:
        plan["violations"].append({
            "constraint": "device_memory", "required_bytes": total, "available_bytes": HBM_BYTES,
            "message": f"weights, cache and workspace need {total} bytes but the device has {HBM_BYTES}",
        })
    return plan


def plan_command(argv: List[str]) -> int:
    args = Args(argv, "plan", {"--json": False, "--ctx": True, "--batch": True, "--dtype": True,
                               "--block-size": True, "--keep-float32": False}, 1)
    if not args.positional:
        raise UsageError("plan needs a model folder")
    dtype = args.values.get("--dtype", "bfloat16")
    if dtype not in ("bfloat16", "float32"):
        raise InvalidArgumentError(f"--dtype expects bfloat16 or float32, got \"{dtype}\"")
    plan = plan_model(args.positional[0], args.number("--ctx", None, int), args.number("--batch", 1, int), dtype,
                      args.number("--block-size", 16, int), "--keep-float32" in args.switches)
    if "--json" in args.switches:
        _emit(json.dumps(plan, indent=2) + "\n")
    else:
        for key, value in plan.items():
            if key != "violations":
                _emit(f"{key}: {value}\n")
        for violation in plan["violations"]:
            _emit(f"violation: {violation['message']}\n")
    return 0 if plan["feasible"] else 3


# --- sample -----------------------------------------------------------------------------------------
def sample_command(argv: List[str]) -> int:
    flags = {"--json": False, "--logits": True, "--logits-file": True, "--count": True, "--seed": True,
             "--temperature": True, "--top-k": True, "--top-p": True, "--min-p": True,
             "--repetition-penalty": True, "--recent": True}
    args = Args(argv, "sample", flags, 0)
    if "--logits" in args.values:
        text = args.values["--logits"]
    elif "--logits-file" in args.values:
        try:
            with open(args.values["--logits-file"]) as handle:
                text = handle.read()
        except OSError as err:
            from .errors import IoError
            raise IoError(f"cannot read {args.values['--logits-file']}: {err.strerror or err}") from None
    else:
        raise UsageError("sample needs --logits or --logits-file")
    try:
        values = [float(part) for part in text.replace(",", " ").split()]
    except ValueError:
        raise InvalidArgumentError("--logits expects numbers separated by commas") from None
    if not values:
        raise InvalidArgumentError("--logits holds no numbers")
    params = _sampling(args, 0.8)
    count = args.number("--count", 1, int)
    recent = _ids(args.values.get("--recent", ""), "--recent")
    import torch

    from .runtime import Runtime
    from .sampling import BatchSampler, RowRequest, seeded_state

    runtime = Runtime("cuda:0", "float32")
    sampler = BatchSampler(runtime.device)
    tokens = []
    for draw in range(count):
        logits = torch.tensor([values], dtype=torch.float32, device=runtime.device)
        row = RowRequest(params, 0, draw, recent, seeded_state(params.seed) if draw == 0 else None)
        token = sampler.sample(logits, [row])[0]
        if token < 0:
            raise InvalidArgumentError("the logits hold no finite value")
        tokens.append(token)
    if "--json" in args.switches:
        _emit(json.dumps({"tokens": tokens, "seed": params.seed, "temperature": params.temperature}) + "\n")
    else:
        _emit(" ".join(str(t) for t in tokens) + "\n")
    return 0


# --- generate ---------------------------------------------------------------------------------------
def generate_command(argv: List[str]) -> int:
    flags = {"--json": False, "--prompt-ids": True, "--prompt-ids-file": True, "--max-tokens": True, "--ctx": True,
             "--dtype": True, "--block-size": True, "--temperature": True, "--top-k": True, "--top-p": True,
             "--min-p": True, "--repetition-penalty": True, "--seed": True, "--keep-float32": False}
    args = Args(argv, "generate", flags, 1)
    if not args.positional:
        raise UsageError("generate needs a model folder")
    if "--prompt-ids" in args.values:
        prompt = _ids(args.values["--prompt-ids"], "--prompt-ids")
    elif "--prompt-ids-file" in args.values:
        try:
            with open(args.values["--prompt-ids-file"]) as handle:
                prompt = _ids(handle.read(), "--prompt-ids-file")
        except OSError as err:
            from .errors import IoError
            raise IoError(f"cannot read {args.values['--prompt-ids-file']}: {err.strerror or err}") from None
    else:
        raise UsageError("generate needs --prompt-ids or --prompt-ids-file")
    max_tokens = args.number("--max-tokens", 32, int)
    if max_tokens < 1:
        raise InvalidArgumentError("--max-tokens must be at least 1")
    dtype = args.values.get("--dtype", "bfloat16")
    if dtype not in ("bfloat16", "float32"):
        raise InvalidArgumentError(f"--dtype expects bfloat16 or float32, got \"{dtype}\"")
    params = _sampling(args, 0.0)  # the command line decodes greedily unless told otherwise (main.rs:557-560)

    from .config.registry import load_config
    from .engine.engine import Engine
    from .errors import UnsupportedError

    folder = args.positional[0]
    config = load_config(folder)
    import torch

    from .models import check_model
    check_model(config, torch.float32 if dtype == "float32" else torch.bfloat16)   # refused before the GPU is touched
    ctx = args.number("--ctx", None, int)
    if ctx is not None and ctx > config.context_limit:
        raise UnsupportedError(f"requested context {ctx} exceeds the model's maximum of {config.context_limit}")
    context = ctx if ctx is not None else min(config.context_limit, 2048)  # main.rs:655-663
    block_size = args.number("--block-size", 16, int)
    # one request at a time, as the reference's command line runs (main.rs:680-693)
    # steps are launched ahead of their tokens (the engine falls back to one step at a time while a request's
    # penalties need its tokens on the host)
    engine = Engine(folder, dtype=dtype, block_size=block_size, max_num_seqs=1, max_model_len=context,
                    num_blocks=(context + block_size - 1) // block_size, pipelined=True,
                    keep_float32="--keep-float32" in args.switches)
    started = time.perf_counter()
    json_out = "--json" in args.switches
    shown = []

    def on_token(token: int) -> None:
        shown.append(token)
        if not json_out:
            _emit(("" if len(shown) == 1 else " ") + str(token))

    request = engine.add_request(prompt, max_tokens, params, on_token=on_token)
    generation = None
    while generation is None:
        report = engine.step()
        for done in report.finished:
            if done.request == request:
                generation = done
    seconds = time.perf_counter() - started
    if generation.finish == "error":
        from .errors import InternalError
        raise InternalError(generation.error or "generation failed")
    if json_out:
        _emit(json.dumps({
            "prompt_tokens": generation.prompt_tokens,
            "processed_tokens": generation.processed_tokens,
            "generated_tokens": len(generation.tokens),
            "finish": generation.finish,
            "tokens": generation.tokens,
            "tokens_per_second": round(len(generation.tokens) / seconds, 2) if seconds > 0 else 0.0,
            "micros": engine.stats()["micros"],
        }, indent=2) + "\n")
    else:
        _emit("\n")
    return 0


# --- random-model ---------------------------------------------------------------------------------
def random_model_command(argv: List[str]) -> int:
    args = Args(argv, "random-model", {"--seed": True, "--dtype": True}, 2)
    if len(args.positional) != 2:
        raise UsageError("random-model needs a config.json and an output folder")
    import torch

    from .config.registry import config_from_dict
    from .models import declare_model
    from .weights import write_random_model

    try:
        with open(args.positional[0]) as handle:
            data = json.load(handle)
    except OSError as err:
        from .errors import IoError
        raise IoError(f"cannot read {args.positional[0]}: {err.strerror or err}") from None
    except json.JSONDecodeError as err:
        from .errors import ParseError
        raise ParseError(f"{args.positional[0]} is not valid JSON: {err}") from None
    dtype = args.values.get("--dtype", "bfloat16")
    if dtype not in ("bfloat16", "float32"):
        raise InvalidArgumentError(f"--dtype expects bfloat16 or float32, got \"{dtype}\"")
    config = config_from_dict(data)
    write_random_model(args.positional[1], config, declare_model(config), args.number("--seed", 0, int),
                       torch.float32 if dtype == "float32" else torch.bfloat16)
    _emit(f"{args.positional[1]}\n")
    return 0


def run(argv: List[str]) -> int:
    if not argv:
        sys.stderr.write(USAGE)
        return 1
    command, rest = argv[0], argv[1:]
    if command in ("--help", "-h", "help"):
        _emit(USAGE)
        return 0
    commands = {
        "model-info": model_info_command, "inspect": model_info_command, "plan": plan_command,
        "sample": sample_command, "generate": generate_command, "random-model": random_model_command,
    }
    if command not in commands:
        raise UsageError(f"unknown command \"{command}\"")
    from . import models  # noqa: F401  (registers architectures and parts)
    return commands[command](rest)


def main(argv: Optional[List[str]] = None) -> int:
    try:
        return run(list(sys.argv[1:] if argv is None else argv))
    except ViperaError as err:
        sys.stderr.write(f"vipera: {err}\n")
        return err.exit_code
    except Exception as err:  # anything unforeseen is an internal error, exit 4
        sys.stderr.write(f"vipera: internal error: {err!r}\n")
        return 4
