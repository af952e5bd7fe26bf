"""The command line, in the reference's manner: ``chat`` generates for given prompts and prints the
tokens, ``bench`` times a run and prints ``key=value`` lines.

Options keep the reference's names and meanings where it has them (examples/cli_common.cpp:44-347):
``--prompt``, ``--prompt-file``, ``--prompt-tokens``, ``--max-new-tokens``, ``--n-ctx``, ``--warmup``,
``--temperature``, ``--top-k``, ``--top-p``, ``--min-p``, ``--repeat-penalty``, ``--repeat-last-n``,
``--presence-penalty``, ``--frequency-penalty``, ``--seed``, ``--output kv|human``, ``--profile``,
``--trace``.  ``--package`` names a
model folder here (``--model`` is the same): there is no packaging step.  New: ``--dtype``, ``--batch``, ``--stop-token-ids``, ``--ignore-eos``,
``--prompt-ids``, ``--prompt-lengths``, ``--random-config`` (random weights from a config.json or a named size),
``--allow-extra-tensors`` (tensors the model does not name are listed and left alone instead of refused).  Options of
the reference that select a backend, offload, vision or speculation have no meaning here and are
refused by the parser.

Text needs the model folder's tokenizer.json and the ``tokenizers`` package; without them prompts and
output are token ids.  In ``--prompt-tokens N`` mode the prompt is N dummy tokens and stopping is off,
as in the reference (examples/bench.cpp:564-583).
"""
from __future__ import annotations

import argparse
import sys
import time
from pathlib import Path

from ..cache import CacheFull
from ..config import config_source
from ..sampling import SamplingError, SamplingParams


def build_parser(prog: str, bench: bool) -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog=prog, description=__doc__.split("\n\n")[0])
    ap.add_argument("--package", "--model", dest="model", help="model folder: config.json + safetensors")
    ap.add_argument("--random-config", "--random", dest="random_config",
                    help="instead of --package: a config.json, or a named size, to fill with random weights")
    ap.add_argument("--allow-extra-tensors", action="store_true",
                    help="load a checkpoint that holds tensors the model does not name (they are listed and left alone)")
    ap.add_argument("--prompt", action="append", default=[], help="prompt text (needs tokenizer.json); may repeat")
    ap.add_argument("--prompt-file", help="read prompt text from a file")
    ap.add_argument("--prompt-ids", action="append", default=[], help="prompt as comma-separated token ids; may repeat")
    ap.add_argument("--prompt-tokens", type=int, default=0, help="use N dummy tokens (no stop token)")
    ap.add_argument("--prompt-lengths", metavar="LO:HI", help="like --prompt-tokens, the length of each of --batch prompts "
                                                              "drawn uniformly from LO..HI (by --seed) and the ids at random")
    ap.add_argument("--batch", type=int, default=1, help="with --prompt-tokens: how many such prompts; else the most "
                                                          "requests in one batch")
    ap.add_argument("--max-new-tokens", type=int, default=2048)
    ap.add_argument("--stop-token-ids", help="comma-separated token ids that end a sequence (default: the model's "
                                             "eos_token_id of config.json and generation_config.json)")
    ap.add_argument("--ignore-eos", action="store_true", help="never stop before --max-new-tokens")
    ap.add_argument("--n-ctx", type=int, default=16384, help="tokens the cache holds for all live sequences together")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--warmup", type=int, default=1, help="warm-up runs before the timed run (bench)")
    ap.add_argument("--temperature", type=float, default=0.6, help="0 = greedy")
    ap.add_argument("--top-k", type=int, default=50, help="0 = disabled")
    ap.add_argument("--top-p", type=float, default=0.9, help="0 = disabled")
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--repeat-penalty", type=float, default=1.0)
    ap.add_argument("--repeat-last-n", type=int, default=64, help="-1 = full context, 0 = disabled")
    ap.add_argument("--presence-penalty", type=float, default=0.0)
    ap.add_argument("--frequency-penalty", type=float, default=0.0)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--output", default="kv", choices=["kv", "human"], help="bench output format")
    ap.add_argument("--profile", action="store_true", help="print time per kernel entry point, prefill and decode apart "
                                                            "(steps then launch kernel by kernel, without HIP graphs)")
    ap.add_argument("--trace", metavar="PATH.json", help="write the steps and kernel launches as a Chrome trace")
    return ap


def sampling_from_args(args) -> SamplingParams:
    p = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
                       repeat_penalty=args.repeat_penalty, repeat_last_n=args.repeat_last_n,
                       presence_penalty=args.presence_penalty, frequency_penalty=args.frequency_penalty, seed=args.seed)
    p.validate()
    return p


def load_tokenizer(model_dir):
    """The folder's tokenizer, or None: text is a convenience, the library's interface is token ids."""
    if model_dir is None:
        return None
    path = Path(model_dir) / "tokenizer.json"
    if not path.is_file():
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(str(path))


def collect_prompts(args, tokenizer, vocab_size: int):
    """Returns (prompts as id lists, stopping disabled?)."""
    if args.prompt_lengths:
        import random
        try:
            lo, hi = (int(x) for x in args.prompt_lengths.split(":"))
        except ValueError:
            raise SystemExit("--prompt-lengths takes LO:HI, two whole numbers")
        if not 1 <= lo <= hi:
            raise SystemExit("--prompt-lengths needs 1 <= LO <= HI")
        rng = random.Random(args.seed)
        lengths = [rng.randint(lo, hi) for _ in range(max(1, args.batch))]
        return [[rng.randrange(vocab_size) for _ in range(n)] for n in lengths], True
    if args.prompt_tokens > 0:
        # token 0 is always valid (examples/bench.cpp:564-567)
        return [[0] * args.prompt_tokens for _ in range(max(1, args.batch))], True
    prompts = []
    for s in args.prompt_ids:
        prompts.append([int(t) for t in s.replace(",", " ").split()])
    texts = list(args.prompt)
    if args.prompt_file:
        texts.append(Path(args.prompt_file).read_text())
    for text in texts:
        if tokenizer is None:
            raise SystemExit("a text prompt needs tokenizer.json in the model folder and the tokenizers package; "
                             "use --prompt-ids")
        prompts.append(tokenizer.encode(text).ids)
    return prompts, False


def make_engine(args):
    from .engine import Engine
    if args.model:
        return Engine.from_dir(args.model, dtype=args.dtype, max_tokens=args.n_ctx, strict_weights=not args.allow_extra_tensors)
    if args.random_config:
        return Engine.from_config(config_source(args.random_config), seed=args.seed, dtype=args.dtype, max_tokens=args.n_ctx)
    raise SystemExit("--package <model folder> (or --random-config <config.json>) is required")


def print_kv(load_ms, m, total_ms, n_requests, finish) -> None:
    """The reference's keys (examples/bench.cpp:190-210)."""
    print(f"load_ms={load_ms:.2f}")
    print(f"requests={n_requests}")
    print(f"prompt_tokens={m.prompt_tokens}")
    print(f"generated_tokens={m.generated_tokens}")
    print(f"decode_tokens={m.decode_tokens}")
    print(f"ttft_ms={m.ttft_ms:.2f}")
    print(f"tpot_ms={m.tpot_ms:.2f}")
    print(f"prefill_tps={m.prefill_tps:.2f}")
    print(f"decode_tps={m.decode_tps:.2f}")
    print(f"prefill_ms={m.ttft_ms:.2f}")
    print(f"decode_ms={m.total_ms - m.ttft_ms:.2f}")
    print(f"total_ms={total_ms:.2f}")
    print(f"hit_eos={int(any(f == 'stop' for f in finish))}")


def print_human(load_ms, m, total_ms, n_requests, finish) -> None:
    print(f"  load      {load_ms:10.1f} ms")
    print(f"  requests  {n_requests:10d}")
    print(f"  prompt    {m.prompt_tokens:10d} tokens   prefill {m.ttft_ms:10.1f} ms   {m.prefill_tps:12.1f} tok/s")
    print(f"  decoded   {m.decode_tokens:10d} tokens   decode  {m.total_ms - m.ttft_ms:10.1f} ms   {m.decode_tps:12.1f} tok/s")
    print(f"  tpot      {m.tpot_ms:10.2f} ms      total   {total_ms:10.1f} ms")


def run(argv, bench: bool) -> int:
    ap = build_parser("palm_bench" if bench else "palm_chat", bench)
    args = ap.parse_args(argv)
    try:
        sampling = sampling_from_args(args)
    except SamplingError as e:
        print(f"{ap.prog}: {e}", file=sys.stderr)
        return 1
    if args.max_new_tokens < 1:
        print(f"{ap.prog}: max_new_tokens must be >= 1", file=sys.stderr)
        return 1
    if args.trace is not None and not args.trace:
        print(f"{ap.prog}: --trace path must not be empty", file=sys.stderr)
        return 1
    t0 = time.perf_counter()
    try:
        engine = make_engine(args)
    except (ValueError, FileNotFoundError, RuntimeError) as e:
        # a config.json, a checkpoint or a build that cannot be used: the message says what and where
        print(f"{ap.prog}: {type(e).__name__}: {e}", file=sys.stderr)
        return 1
    load_ms = (time.perf_counter() - t0) * 1000.0
    tokenizer = load_tokenizer(args.model)
    prompts, no_stop = collect_prompts(args, tokenizer, engine.vocab_size)

    no_stop = no_stop or args.ignore_eos
    stop_ids = None
    if args.stop_token_ids is not None:
        try:
            stop_ids = tuple(int(t) for t in args.stop_token_ids.replace(",", " ").split())
        except ValueError:
            print(f"{ap.prog}: --stop-token-ids takes comma-separated whole numbers", file=sys.stderr)
            return 1
    if not bench and not prompts:
        return repl(engine, sampling, tokenizer, args, stop_ids)
    if not prompts:
        prompts = [[0] * 16]
        no_stop = True
    try:
        return _generate_and_report(ap, args, engine, sampling, tokenizer, prompts, stop_ids, no_stop, load_ms, bench)
    except (ValueError, CacheFull) as e:
        # a prompt that does not fit the cache, a token outside the vocabulary
        print(f"{ap.prog}: {type(e).__name__}: {e}", file=sys.stderr)
        return 1


def _generate_and_report(ap, args, engine, sampling, tokenizer, prompts, stop_ids, no_stop, load_ms, bench) -> int:
    if bench:
        for _ in range(max(0, args.warmup)):
            engine.generate(prompts, sampling, args.max_new_tokens, stop_token_ids=stop_ids, ignore_eos=no_stop,
                            max_batch=max(1, args.batch))
    recorder = None
    if args.profile or args.trace:
        # after the warm-up, so that what is timed has loaded its libraries and the tables show the timed run alone
        from ..kernels.profile import KernelProfile
        recorder = KernelProfile().install()
    t1 = time.perf_counter()

    def stream(i, tok):
        if not bench and len(prompts) == 1:
            piece = tokenizer.decode([tok]) if tokenizer else f"{tok} "
            print(piece, end="", flush=True)

    try:
        results, metrics = engine.generate(prompts, sampling, args.max_new_tokens, stop_token_ids=stop_ids,
                                           ignore_eos=no_stop, max_batch=max(1, args.batch), on_token=stream)
    finally:
        if recorder is not None:
            recorder.remove()
    total_ms = (time.perf_counter() - t1) * 1000.0
    if args.trace:
        recorder.write_chrome_trace(args.trace)
    if bench:
        (print_human if args.output == "human" else print_kv)(load_ms, metrics, total_ms, len(prompts),
                                                               [r.finish_reason for r in results])
        if args.profile:
            print(recorder.format())
        return 0
    if len(prompts) == 1:
        print()
    else:
        for i, r in enumerate(results):
            text = tokenizer.decode(r.token_ids) if tokenizer else " ".join(map(str, r.token_ids))
            print(f"[{i}] {text}")
    if args.profile:
        print(recorder.format(), file=sys.stderr)
    print(f"ttft {metrics.ttft_ms:.1f} ms | tpot {metrics.tpot_ms:.2f} ms | prefill {metrics.prefill_tps:.1f} tok/s | "
          f"decode {metrics.decode_tps:.1f} tok/s | tokens {metrics.generated_tokens}", file=sys.stderr)
    return 0


def repl(engine, sampling, tokenizer, args, stop_ids=None) -> int:
    """Turns from standard input, one a line (text with a tokenizer, else token ids).  The conversation stays in
    the cache: a turn feeds only its own tokens on top of what earlier turns left (examples/main.cpp:394-466);
    ``/reset`` starts over, ``/quit`` ends (examples/main.cpp:524-548)."""
    print("one turn a line; /reset to start over, /quit to end", file=sys.stderr)
    talk = engine.conversation(sampling, stop_token_ids=stop_ids, ignore_eos=args.ignore_eos)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        if line == "/reset":
            talk.reset()
            continue
        if line in ("/quit", "/exit"):
            break
        try:
            ids = tokenizer.encode(line).ids if tokenizer else [int(t) for t in line.replace(",", " ").split()]
        except ValueError:
            print("without a tokenizer a turn is a list of token ids", file=sys.stderr)
            continue
        try:
            result = talk.say(ids, args.max_new_tokens)
        except (ValueError, CacheFull) as e:
            print(f"{type(e).__name__}: {e}", file=sys.stderr)
            continue
        out = result.token_ids
        print(tokenizer.decode(out) if tokenizer else " ".join(map(str, out)), flush=True)
    talk.reset()
    return 0


def chat_main(argv=None) -> int:
    return run(sys.argv[1:] if argv is None else argv, bench=False)


def bench_main(argv=None) -> int:
    return run(sys.argv[1:] if argv is None else argv, bench=True)
