"""Command line in the manner of the reference's ``burn-lm`` (crates/burn-lm-cli/src/cli.rs:5-69):
with no command it opens the shell; ``models`` lists what can be run; ``run <model> [flags]
<prompt>`` generates once and prints the stats table; ``chat <model> [flags]`` is an interactive
session with the slash commands ``/help /stats /clear /exit``; ``-d/--dtype`` picks the element
type (a run-time choice here, a recompilation there).  ``random <preset>`` stands where
``download`` does in the reference: it puts a model folder with seeded random weights into the
models directory; ``delete <model>|all`` removes folders from it.  A model is named by a folder path or by a folder name inside the models
directory (``$BURN_LM_AMD_MODELS``, default ``~/.cache/burn-lm_amd/models``).
"""
from __future__ import annotations

import argparse
import os
import shlex
import sys

from ..config.presets import preset, presets
from ..server import InferenceServer, add_cli_flags

BACKEND = "gfx950"


def models_dir():
    return os.environ.get("BURN_LM_AMD_MODELS") or os.path.join(os.path.expanduser("~"), ".cache", "burn-lm_amd", "models")


def resolve_model(name):
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return name
    cand = os.path.join(models_dir(), name)
    if os.path.exists(os.path.join(cand, "config.json")):
        return cand
    raise SystemExit(f"model {name!r} not found: give a folder with config.json and model.safetensors, or create one "
                     f"with `random <preset>` (models directory: {models_dir()})")


def build_parser():
    p = argparse.ArgumentParser(prog="burn-lm-amd", description="Run language models on an MI355X.")
    p.add_argument("-b", "--backend", default=BACKEND, help="The backend selected (only gfx950).")
    p.add_argument("-d", "--dtype", default="bf16", choices=["bf16", "f32", "bfloat16", "float32"],
                   help="The element type used.")
    sub = p.add_subparsers(dest="command")
    sub.add_parser("models", help="List the models that can be run and the presets for random weights")
    sub.add_parser("backends", help="List the backends (there is one)")
    r = sub.add_parser("run", help="Run inference on chosen model in the terminal")
    r.add_argument("model")
    add_cli_flags(r)
    r.add_argument("--no-stats", action="store_true", help="Disable display of statistics at the end of the inference")
    r.add_argument("--tokens", action="store_true", help="Every prompt is a comma-separated list of token ids")
    r.add_argument("--batch", type=int, default=None, metavar="N",
                   help="Sequences that run together (default: as many as there are prompts, at most 64); "
                        "more prompts than that run batch after batch")
    r.add_argument("--prompts-file", default=None, metavar="FILE", help="More prompts, one a line")
    r.add_argument("--cast-32bit", action="store_true",
                   help="Round matrices that the checkpoint stores in 32 bits to the element type when loading")
    r.add_argument("prompt", nargs="*", help="The prompt to send to the model; several prompts run as one batch "
                                             "of unequal lengths, and one line per request is printed")
    c = sub.add_parser("chat", help="Start a chat session with the chosen model")
    c.add_argument("model")
    add_cli_flags(c)
    g = sub.add_parser("random", help="Write a model folder with seeded random weights for a preset")
    g.add_argument("preset")
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--name", default=None, help="folder name inside the models directory (default: the preset's)")
    g.add_argument("--layers", type=int, default=None, help="override the number of layers")
    dl = sub.add_parser("delete", help="Delete models from the models directory")
    dl.add_argument("model", help="a folder name inside the models directory, or 'all'")
    sub.add_parser("shell", help="Start a burn-lm-amd shell session")
    return p


def cmd_models():
    d = models_dir()
    rows = []
    if os.path.isdir(d):
        for n in sorted(os.listdir(d)):
            if os.path.exists(os.path.join(d, n, "config.json")):
                rows.append((n, "yes", f"run {n} \"<prompt>\""))
    for n in sorted(presets()):
        if not any(r[0] == n for r in rows):
            rows.append((n, "no", f"random {n}"))
    w = [max(len(r[i]) for r in rows + [("Model", "Present", "Command")]) for i in range(3)]
    print(f"| {'Model':<{w[0]}} | {'Present':<{w[1]}} | {'Command':<{w[2]}} |")
    print(f"|{'-' * (w[0] + 2)}|{'-' * (w[1] + 2)}|{'-' * (w[2] + 2)}|")
    for r in rows:
        print(f"| {r[0]:<{w[0]}} | {r[1]:<{w[1]}} | {r[2]:<{w[2]}} |")


def cmd_random(args):
    from ..weights.random_init import write_model_folder
    cfg = preset(args.preset)
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    folder = os.path.join(models_dir(), args.name or args.preset)
    print(f"writing random weights (seed {args.seed}) for {args.preset} into {folder} ...")
    write_model_folder(folder, cfg, seed=args.seed)
    print("done")


def cmd_delete(args):
    """``delete <model>|all`` (crates/burn-lm-cli/src/commands/delete.rs:4-23): removes model folders,
    and only those of the models directory, one after the other."""
    import shutil
    d = models_dir()
    present = sorted(n for n in (os.listdir(d) if os.path.isdir(d) else [])
                     if os.path.exists(os.path.join(d, n, "config.json")))
    names = present if args.model == "all" else [args.model]
    for n in names:
        if n not in present or os.sep in n or n in (".", ".."):
            raise SystemExit(f"model {n!r} is not in the models directory {d} (it holds: {', '.join(present) or 'nothing'})")
    for n in names:
        print(f"deleting model '{n}'...")
        shutil.rmtree(os.path.join(d, n))
        print("model deleted!")
    if not names:
        print("no model to delete")


def cmd_run(args):
    """``run <model> [flags] <prompt>`` (crates/burn-lm-cli/src/commands/run.rs:7-97: load, generate,
    print the text as it comes, then the stats table).  Several prompts (more arguments, or the lines
    of --prompts-file) run as batches of unequal lengths; each request then gets a line of its own."""
    prompts = list(args.prompt)
    if args.prompts_file:
        with open(args.prompts_file) as f:
            prompts += [line.rstrip("\n") for line in f if line.strip()]
    if not prompts:
        raise SystemExit("run: give a prompt (or several, or --prompts-file)")
    batch = args.batch or min(len(prompts), 64)
    if batch < 1:
        raise SystemExit("run: --batch must be at least 1")
    server = InferenceServer(resolve_model(args.model), dtype=args.dtype, batch_size=batch, cast_32bit=args.cast_32bit)
    server.parse_cli_config(args)
    print(f"loading model '{server.model_name()}'...", file=sys.stderr)
    server.load()
    print("model loaded!", file=sys.stderr)
    if args.tokens:
        try:
            ids = [[int(t) for t in p.replace(",", " ").split()] for p in prompts]
        except ValueError as e:
            raise SystemExit(f"run --tokens: a prompt is no list of token ids ({e})") from None
        results, stats = server.generate(ids)
        for r in results:
            if r.finish_reason == "error" and len(results) == 1:
                raise SystemExit(r.error)
            print(",".join(str(t) for t in r.tokens) if r.finish_reason != "error" else f"error: {r.error}")
    elif len(prompts) == 1:
        stats = server.run_job({"role": "user", "content": prompts[0]},
                               on_text=lambda s: (sys.stdout.write(s), sys.stdout.flush()))
        print()
    else:
        texts, stats = server.run_jobs([{"role": "user", "content": p} for p in prompts])
        for i, t in enumerate(texts):
            print(f"[{i}] {t}")
    stats.model_loading_seconds = server._load_seconds
    if not args.no_stats:
        print(stats.display_stats())
    server.unload()


def cmd_chat(args):
    server = InferenceServer(resolve_model(args.model), dtype=args.dtype, batch_size=1)
    server.parse_cli_config(args)
    print(f"loading model '{server.model_name()}'...", file=sys.stderr)
    server.load()
    print("model loaded!", file=sys.stderr)
    show_stats = True
    print("Chat session started! (press CTRL+D or type /exit to close session)")
    prompt = f"({BACKEND}-{args.dtype}) chat|{server.model_name()}> "
    while True:
        try:
            line = input(prompt).strip()
        except EOFError:
            break
        if not line:
            continue
        if line.startswith("/"):  # slash commands of crates/burn-lm-cli/src/commands/chat.rs:13-27
            cmd = line[1:].split()[0] if len(line) > 1 else ""
            if cmd == "exit":
                break
            if cmd == "help":
                print("/help   show this help\n/stats  toggle the stats table\n/clear  clear the chat state\n/exit   close the session")
            elif cmd == "stats":
                show_stats = not show_stats
                print(f"Stats toggled {'on' if show_stats else 'off'}!")
            elif cmd == "clear":
                server.clear_state()
                print("Chat state cleared!")
            else:
                print(f"unknown command /{cmd}; try /help")
            continue
        try:
            stats = server.run_job({"role": "user", "content": line},
                                   on_text=lambda s: (sys.stdout.write(s), sys.stdout.flush()))
        except Exception as e:
            print(f"An error occurred: {e}")
            continue
        print()
        if show_stats:
            print(stats.display_stats())
    server.unload()
    print("Chat session closed!")


def cmd_shell(dtype):
    parser = build_parser()
    print("Welcome to the burn-lm-amd shell (press CTRL+D or type 'exit' to close)")
    while True:
        try:
            line = input(f"({BACKEND}-{dtype}) burnlm> ").strip()
        except EOFError:
            break
        if not line:
            continue
        if line in ("exit", "quit"):
            break
        try:
            args = parse(parser, ["-d", dtype] + shlex.split(line))
            if args.command in (None, "shell"):
                parser.print_help()
            else:
                dispatch(args)
        except SystemExit as e:
            if e.code not in (0, None):
                print(e)
        except Exception as e:
            print(f"An error occurred: {e}")


def dispatch(args):
    if args.command == "models":
        cmd_models()
    elif args.command == "backends":
        print(f"{BACKEND} (HIP, MI355X) [selected]")
    elif args.command == "run":
        cmd_run(args)
    elif args.command == "chat":
        cmd_chat(args)
    elif args.command == "random":
        cmd_random(args)
    elif args.command == "delete":
        cmd_delete(args)


def parse(parser, argv):
    """argparse gives a sub-command's list of positionals only what stands in front of its first
    flag; prompts that come after flags are picked up here."""
    args, rest = parser.parse_known_args(argv)
    if rest:
        if args.command != "run" or any(r.startswith("-") for r in rest):
            parser.error("unrecognized arguments: " + " ".join(rest))
        args.prompt = list(args.prompt) + rest
    return args


def main(argv=None):
    args = parse(build_parser(), argv)
    if args.backend != BACKEND:
        raise SystemExit(f"backend {args.backend!r} is not available; this build has {BACKEND} only")
    args.dtype = {"bf16": "bf16", "bfloat16": "bf16", "f32": "f32", "float32": "f32"}[args.dtype]
    if args.command in (None, "shell"):  # the default command is the shell (cli.rs:65-68)
        cmd_shell(args.dtype)
    else:
        dispatch(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
