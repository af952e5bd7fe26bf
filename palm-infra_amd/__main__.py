"""``python -m palm_infra_amd <command> [options]``: the programs under ``bin/`` by name.

    chat          generate for given prompts (bin/palm_chat)
    bench         time a run, ``key=value`` lines (bin/palm_bench)
    random-model  write a model folder with random weights (bin/palm_random_model)
    trace-run     replay given token ids step by step and write logits (bin/trace_run)
"""
import sys


def main(argv=None) -> int:
    argv = sys.argv[1:] if argv is None else list(argv)
    commands = ("chat", "bench", "random-model", "trace-run")
    if not argv or argv[0] in ("-h", "--help") or argv[0] not in commands:
        print(__doc__.strip(), file=sys.stderr if argv and argv[0] not in ("-h", "--help") else sys.stdout)
        return 0 if argv and argv[0] in ("-h", "--help") else 2
    command, rest = argv[0], argv[1:]
    if command == "chat":
        from .engine.cli import chat_main
        return chat_main(rest)
    if command == "bench":
        from .engine.cli import bench_main
        return bench_main(rest)
    if command == "random-model":
        from .weights.random_init import main as random_main
        return random_main(rest)
    from .engine.trace import main as trace_main
    return trace_main(rest)


if __name__ == "__main__":
    raise SystemExit(main())
