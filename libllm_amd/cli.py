"""The command line, in the manner of the reference's ``llm`` program (go/bin/main.go:27-54,
go/bin/args.go:54-91, go/bin/chat.go:44-132): ``llm chat -m MODEL -device cpu|cuda|auto`` opens a
prompt loop with ``:new`` (clear the history), ``:sys <prompt>`` (set the system prompt and clear),
empty lines ignored and end of input leaving; after each reply it prints
``(N tokens, time=..s, ..ms per token)``.  Flags take one or two dashes.  ``llm benchmark`` is the
counterpart of the reference's llm_benchmark (src/libllm/benchmark_main.cc:98-134).

Tokenisation is outside this library: with ``-ids`` a line is a list of token ids and the reply is
printed as ids; otherwise a tokenizer.json beside the model, or bytes as token ids, are used.  The
session's messages go into the architecture's chat format (``Model.build_prompt``,
src/libllm/llama.cc:406-442) where that tokenizer knows its control tokens, else as lines of text.
"""
import argparse
import sys
import time

from .errors import LlmError

MSG_INPUT = "Please input your question."
MSG_NEW = "    Type ':new' to start a new session (clean history)."
MSG_SYS = "    Type ':sys <system_prompt>' to set the system prompt and start a new session ."
MSG_NEW_SESSION = "===== new session ====="
MSG_STAT = "(%d tokens, time=%.2fs, %.2fms per token)"


def _usage():
    sys.stderr.write("Usage: llm COMMAND\n\nCommands:\n"
                     "    chat           Chat with LLM\n"
                     "    benchmark      Measure prompt and decoding speed\n\n"
                     "Run 'llm COMMAND -h' for more information on a command.\n")


def _flag(ap, name, **kw):
    ap.add_argument("-" + name, "--" + name.replace("_", "-"), dest=name, **kw)


def _model_args(prog):
    ap = argparse.ArgumentParser(prog=prog, allow_abbrev=False)
    _flag(ap, "m", action="append", default=[], metavar="MODEL",
          help="the model folder (config.json and model.safetensors)")
    _flag(ap, "device", default="auto", help="inference device, either cpu, cuda (or hip) or auto")
    _flag(ap, "dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"])
    _flag(ap, "random_weights", action="store_true",
          help="read only config.json from the model folder and draw the weights from -seed")
    _flag(ap, "max_tokens", type=int, default=8192, help="tokens the cache holds")
    return ap


def _load(args, ap):
    device = args.device.lower()
    if device not in ("cpu", "cuda", "hip", "auto"):
        ap.error('invalid device name: must be one of "cpu", "cuda" or "auto"')
    if len(args.m) == 0:
        ap.error("model name (-m) is empty.")
    if len(args.m) != 1:
        ap.error("only 1 model (-m) is expected")
    from .api import Model
    return Model(args.m[0], device, dtype=args.dtype, max_tokens=args.max_tokens,
                 random_weights=args.random_weights, seed=getattr(args, "seed", 0))


def chat_main(argv) -> int:
    ap = _model_args("llm chat")
    _flag(ap, "temperature", type=float, default=1.0)
    _flag(ap, "top_k", type=int, default=50)
    _flag(ap, "top_p", type=float, default=0.8)
    _flag(ap, "seed", type=int, default=0, help="seed of the sampler (and of -random_weights)")
    _flag(ap, "max_new_tokens", type=int, default=256)
    _flag(ap, "ids", action="store_true", help="lines are token ids; replies are printed as ids")
    _flag(ap, "stop_id", type=int, action="append", default=None,
          help="a token id that ends a reply, beside the model's own (repeatable)")
    args = ap.parse_args(argv)
    model = _load(args, ap)
    print(MSG_INPUT)
    print(MSG_NEW)
    print(MSG_SYS)
    history = []                 # token ids of the session so far (with -ids) or (role, text) pairs
    system_prompt = ""
    turn = 0
    while True:
        sys.stdout.write("> ")
        sys.stdout.flush()
        line = sys.stdin.readline()
        if line == "":
            print()
            break
        question = line.strip()
        if len(question) > 5 and question[:5].lower() == ":sys ":
            system_prompt = question[5:].strip()
            history = []
            continue
        if question.lower() == ":new":
            print(MSG_NEW_SESSION)
            history = []
            continue
        if question == "":
            continue
        if args.ids:
            try:
                ids = [int(t) for t in question.replace(",", " ").split()]
            except ValueError:
                print("with -ids a line must hold token ids")
                continue
            prompt = history + ids
        else:
            if not history and system_prompt:
                history.append(("system", system_prompt))
            history.append(("user", question))
            prompt = model.build_prompt([{"role": role, "content": text} for role, text in history])
        t0 = time.time()
        n, reply_ids, reply_text = 0, [], ""
        for chunk in model.complete(prompt, top_k=args.top_k, top_p=args.top_p, temperature=args.temperature,
                                    max_new_tokens=args.max_new_tokens, seed=args.seed + turn,
                                    stop_ids=(args.stop_id or []) + ([] if args.ids else model.chat_stop_ids())):
            if chunk.token_id is not None:
                n += 1
                reply_ids.append(chunk.token_id)
            text = (str(chunk.token_id) + " ") if args.ids else chunk.text
            if args.ids and chunk.token_id is None:
                continue
            reply_text += chunk.text
            sys.stdout.write(text)
            sys.stdout.flush()
        print()
        if args.ids:
            history = prompt + reply_ids
        else:
            history.append(("assistant", reply_text))
        dur = time.time() - t0
        print(MSG_STAT % (n, dur, dur * 1000.0 / max(n, 1)))
        turn += 1
    return 0


def benchmark_main(argv) -> int:
    """Prompt and decoding speed of one sequence, as the reference's tool reports them
    (src/libllm/benchmark_main.cc:52-86): tokens per second of a prompt of ``-l`` tokens and of
    single tokens decoded after it."""
    ap = _model_args("llm benchmark")
    _flag(ap, "l", type=int, default=512, help="prompt length in tokens")
    _flag(ap, "n", type=int, default=64, help="decoded tokens")
    args = ap.parse_args(argv)
    model = _load(args, ap)
    import torch
    from .engine import StepEntry
    vocab = model.engine.vocab
    prompt = [(7 * i + 3) % vocab for i in range(args.l)]
    for _ in range(2):
        t0 = time.time()
        model.step([StepEntry("bench", prompt, [len(prompt) - 1])])
        torch.cuda.synchronize()
        prefill = time.time() - t0
        t0 = time.time()
        for i in range(args.n):
            model.step([StepEntry("bench", [i % vocab], [0])])
        torch.cuda.synchronize()
        decode = time.time() - t0
        model.end(["bench"])
    print("prefill@%d  %.1f tokens/s" % (args.l, args.l / prefill))
    print("decode@%d   %.1f tokens/s" % (args.l, args.n / decode))
    ops = model.engine.ops
    if getattr(ops, "timing", False):                       # LIBLLM_AMD_TIME=1: where the time went
        for name, calls, ms in ops.timing_report():
            print("  %-14s %6d calls %10.3f ms" % (name, calls, ms))
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv:
        _usage()
        return 1
    command, rest = argv[0], argv[1:]
    try:
        if command == "chat":
            return chat_main(rest)
        if command in ("benchmark", "bench"):
            return benchmark_main(rest)
    except LlmError as e:
        sys.stderr.write("llm: %s\n" % e)
        return 1
    sys.stderr.write('Invalid command "%s"\n\n' % command)
    _usage()
    return 1
