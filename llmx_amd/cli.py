"""The command line, in the reference's manner (/root/reference/src/cli/main.cpp): `llmx generate MODEL [PROMPT]`.

Flags keep the reference's names and meanings where it has them (main.cpp:2018-2038 sampling, :541-574 execution):
--max-tokens/-n, --temp, --topk, --topp, --min-p, --penalty, --presence-penalty, --frequency-penalty, --seed,
--ignore-eos, --stop, --dtype, --ubatch, --kv-tokens, --verbose; logits: --then-ids, --last, --per-token, --top;
perplexity: --ctx-size/-c, --chunks, --per-token.  There is no tokenizer here: a prompt is a list of token ids
(comma or space separated), given on the line, with --file, or made up with --prompt-len; a stop text is a sequence
of token ids.  Instead of a model folder, `--config JSON --random SEED` runs the configuration with weights generated
on the device from the seed (the reference builds its file-less model the same way for its bench,
/root/reference/src/model/arch/registry.hpp:144-152): `llmx generate --config cfg.json --random 0 "1 2 3"`.
A usage error exits with status 2 (main.cpp:100-103); a flag given twice is refused (:129-159).
"""

from __future__ import annotations

import argparse
import json
import re
import sys
import time
from pathlib import Path


class _Once(argparse.Action):
    """A second value for the same setting is refused rather than overwriting the first."""

    def __call__(self, parser, namespace, values, option_string=None):
        seen = getattr(namespace, "_given", set())
        if self.dest in seen:
            parser.error(f"{option_string}: given twice")
        seen.add(self.dest)
        namespace._given = seen
        setattr(namespace, self.dest, True if self.nargs == 0 else values)


def _add_sampling(p):
    from .sampling.params import SamplingParams
    d = SamplingParams()
    p.add_argument("--max-tokens", "-n", type=int, default=d.max_tokens, action=_Once, help="tokens generated at most (default %(default)s)")
    p.add_argument("--temp", type=float, default=d.temp, action=_Once, help="temperature, 0 is greedy (default %(default)s)")
    p.add_argument("--topk", type=int, default=d.top_k, action=_Once, help="keep the k likeliest tokens, 0 keeps all (default %(default)s)")
    p.add_argument("--topp", type=float, default=d.top_p, action=_Once, help="nucleus share of the kept weight (default %(default)s)")
    p.add_argument("--min-p", type=float, default=d.min_p, action=_Once, help="drop tokens below this share of the likeliest (default %(default)s)")
    p.add_argument("--penalty", type=float, default=d.penalty, action=_Once, help="repetition penalty, 1 is none (default %(default)s)")
    p.add_argument("--presence-penalty", type=float, default=d.presence_penalty, action=_Once)
    p.add_argument("--frequency-penalty", type=float, default=d.frequency_penalty, action=_Once)
    p.add_argument("--seed", type=int, default=d.seed, action=_Once, help="0 keeps the fixed default generator state")
    p.add_argument("--ignore-eos", nargs=0, default=False, action=_Once, help="the end token is never drawn")
    p.add_argument("--stop", default="", action=_Once, help="token ids; generation ends when the generated ids end with them")


def _add_exec(p):
    p.add_argument("--dtype", choices=["f32", "bf16", "float32", "bfloat16"], default="bf16", action=_Once,
                   help="bf16: the serving path; f32: everything in true 32-bit")
    p.add_argument("--device", default="cuda:0", action=_Once, help="the GPU to run on (default %(default)s)")
    p.add_argument("--cache-type-k", "-ctk", choices=["f32", "bf16", "f16"], default=None, action=_Once,
                   help="type of the cached keys: the type of --dtype (the attention kernels read q, k and v in one type)")
    p.add_argument("--cache-type-v", "-ctv", choices=["f32", "bf16", "f16"], default=None, action=_Once, help="type of the cached values: as --cache-type-k")
    p.add_argument("--ubatch", type=int, default=512, action=_Once, help="tokens a step takes at most (default %(default)s)")
    p.add_argument("--kv-tokens", type=int, default=0, action=_Once, help="the cache's token budget; 0 sizes it to the run")
    p.add_argument("--page-tokens", type=int, default=16, action=_Once, help="tokens a cache page holds (default %(default)s)")
    p.add_argument("--max-seqs", type=int, default=8, action=_Once, help="requests running together at most (default %(default)s)")
    p.add_argument("--verbose", nargs=0, default=False, action=_Once)
    p.add_argument("--config", default=None, action=_Once, help="a config.json to run with random weights instead of a model folder (needs --random)")
    p.add_argument("--random", type=int, default=None, action=_Once, help="seed of the weights generated on the device for --config")
    p.add_argument("--std", type=float, default=0.02, action=_Once, help="standard deviation of the random matrices (default %(default)s)")


def _model_and_prompt(a, command: str):
    """The positionals are MODEL [PROMPT], or [PROMPT] alone when --config names the model."""
    words = list(a.words)
    short = {"float32": "f32", "bfloat16": "bf16"}.get(a.dtype, a.dtype)
    for flag, value in (("--cache-type-k", a.cache_type_k), ("--cache-type-v", a.cache_type_v)):
        if value is not None and value != short:
            raise SystemExit2(f"{flag} {value}: the cache is kept in the type of the activations (--dtype {short}); another cache type is not built")
    if not re.fullmatch(r"cuda(:\d+)?", a.device):
        raise SystemExit2(f"--device {a.device}: this engine runs on a GPU only (cuda or cuda:N)")
    if (a.config is None) != (a.random is None):
        raise SystemExit2(f"{command}: --config and --random go together")
    if a.config is None:
        if not words:
            raise SystemExit2(f"{command} needs a model folder, or --config JSON --random SEED")
        a.model, words = words[0], words[1:]
    else:
        a.model = None
    if len(words) > 1:
        raise SystemExit2(f"{command}: unexpected argument {words[1]!r}")
    a.prompt = words[0] if words else None


def _config_of(a):
    from .models import read_config, read_model_dir
    if a.model is not None:
        return read_model_dir(a.model)[0]
    try:
        return read_config(json.loads(Path(a.config).read_text()))
    except (OSError, json.JSONDecodeError) as e:
        raise SystemExit2(f"--config {a.config}: {e}")


def _engine(a, cfg, **options):
    """The engine of the model folder, or of the configuration with weights generated on the device."""
    from .engine import Engine
    options["device"] = a.device
    if a.model is not None:
        return Engine.load(a.model, dtype=a.dtype, **options)
    from .weights import RandomInit
    return Engine.from_random(cfg, RandomInit(seed=a.random, std=a.std), dtype=a.dtype, **options)


def _ids(text: str):
    parts = [t for t in re.split(r"[,\s]+", text.strip()) if t]
    try:
        return [int(t) for t in parts]
    except ValueError:
        raise SystemExit2(f"a prompt is a list of token ids, not {text[:40]!r}")


class SystemExit2(Exception):
    pass


def _params(a):
    from .sampling.params import SamplingParams
    return SamplingParams(max_tokens=a.max_tokens, temp=a.temp, top_k=a.topk, top_p=a.topp, min_p=a.min_p, penalty=a.penalty,
                          presence_penalty=a.presence_penalty, frequency_penalty=a.frequency_penalty, seed=a.seed,
                          ignore_eos=bool(a.ignore_eos), stop=tuple(_ids(a.stop)) if a.stop else ()).validate()


def _lcg_ids(n: int, vocab: int, seed: int = 1):
    """Fixed token ids spread over the vocabulary (the reference's bench ids, main.cpp:1185-1189, are an LCG too)."""
    x, out = seed & 0xFFFFFFFF, []
    for _ in range(n):
        x = (x * 1664525 + 1013904223) & 0xFFFFFFFF
        out.append((x >> 8) % vocab)
    return out


def cmd_generate(a) -> int:
    from .engine.generation import Generator
    from .engine.scheduler import Request
    _model_and_prompt(a, "generate")
    params = _params(a)
    cfg = _config_of(a)
    if a.file:
        prompts = [_ids(line) for line in Path(a.file).read_text().splitlines() if line.strip()]
    elif a.prompt is not None:
        prompts = [_ids(a.prompt)]
    elif a.prompt_len:
        prompts = [_lcg_ids(a.prompt_len, cfg.vocab_size)]
    else:
        raise SystemExit2("generate needs a prompt: token ids on the line, --file, or --prompt-len")
    if any(not p for p in prompts):
        raise SystemExit2("generate: empty prompt")
    need = sum(len(p) + params.max_tokens for p in prompts[:a.max_seqs]) if len(prompts) > 1 else len(prompts[0]) + params.max_tokens
    kv_tokens = a.kv_tokens or max(need + a.page_tokens * a.max_seqs, max(len(p) for p in prompts) + params.max_tokens)
    engine = _engine(a, cfg, kv_tokens=kv_tokens, page_tokens=a.page_tokens, max_requests=a.max_seqs, step_tokens=a.ubatch)
    gen = Generator(engine, a.max_seqs, a.ubatch)
    for i, p in enumerate(prompts):
        import copy
        gen.submit(Request(i, p, copy.copy(params)))
    if a.verbose:
        print(f"prompt tokens: {sum(len(p) for p in prompts)}")
    import torch
    finished = gen.run()
    torch.cuda.synchronize()
    for i in range(len(prompts)):
        print(" ".join(str(t) for t in finished[i].generated))
    st = gen.stats
    pp_ms, tg_ms = st.prompt_seconds * 1e3, st.decode_seconds * 1e3
    print(f"pp: {st.prompt_tokens} tok, {pp_ms:.0f} ms, {st.prompt_tokens / max(pp_ms, 1e-9) * 1e3:.2f} tok/s", file=sys.stderr)
    print(f"tg: {st.generated_tokens} tok, {tg_ms:.0f} ms, {st.generated_tokens / max(tg_ms, 1e-9) * 1e3:.2f} tok/s", file=sys.stderr)
    if a.verbose:
        print(f"kv: allocated {engine.cache_bytes()} bytes", file=sys.stderr)
        for i in range(len(prompts)):
            print("ids: " + ",".join(str(t) for t in finished[i].generated) + f"  ({finished[i].finish_reason})", file=sys.stderr)
    return 0


def cmd_logits(a) -> int:
    """Top-N logits of the last positions, whole or token by token (the reference's `llmx logits`, main.cpp:934-980)."""
    from .engine import StepEntry
    _model_and_prompt(a, "logits")
    ids = _prompt_ids(a, "logits")
    if a.then_ids:
        ids = ids + _ids(Path(a.then_ids).read_text())
    if not ids:
        raise SystemExit2("logits: empty prompt")
    engine = _engine(a, _config_of(a), kv_tokens=a.kv_tokens or len(ids) + a.page_tokens, page_tokens=a.page_tokens, max_requests=1)
    engine.add_request(0)
    last = min(a.last or 1, len(ids))
    rows = []
    if a.per_token:
        for i, t in enumerate(ids):
            lg = engine.step([StepEntry(0, [t], [0])])
            if i >= len(ids) - last:
                rows.append(lg[0].clone())
    else:
        for s in range(0, len(ids), a.ubatch):
            part = ids[s:s + a.ubatch]
            want = [i - s for i in range(max(s, len(ids) - last), s + len(part))]
            lg = engine.step([StepEntry(0, part, want)])
            rows.extend(r.clone() for r in lg)
    print(f"tokens: {len(ids)}")
    for off, row in enumerate(rows):
        vals, idx = row.topk(min(a.top, row.numel()))
        if a.last:          # one line a position: the position, then id and logit of each of the top
            print(f"{len(ids) - len(rows) + off} " + " ".join(f"{int(i)} {float(v):.6f}" for v, i in zip(vals, idx)))
        else:               # the last position alone: one line for each of the top
            for v, i in zip(vals, idx):
                print(f"{int(i)} {float(v):.6f}")
    return 0


def _prompt_ids(a, command: str):
    if a.prompt is not None and a.file:
        raise SystemExit2(f"{command}: token ids on the line or --file, not both")
    if a.prompt is not None:
        return _ids(a.prompt)
    if a.file:
        return _ids(Path(a.file).read_text())
    if getattr(a, "then_ids", None):
        return []
    raise SystemExit2(f"{command} needs token ids: on the line or with --file")


def cmd_perplexity(a) -> int:
    """Mean negative log-likelihood over windows of token ids (the reference's `llmx perplexity`, main.cpp:982-1008)."""
    from .engine.perplexity import MIN_WINDOW, perplexity
    _model_and_prompt(a, "perplexity")
    ids = _prompt_ids(a, "perplexity")
    if len(ids) < MIN_WINDOW:
        raise SystemExit2(f"perplexity: need at least {MIN_WINDOW} tokens")
    window = min(a.ctx_size or len(ids), len(ids))
    engine = _engine(a, _config_of(a), kv_tokens=a.kv_tokens or window + a.page_tokens, page_tokens=a.page_tokens, max_requests=1)
    window = min(window, engine.max_positions)
    r = perplexity(engine, ids, window, a.chunks, a.per_token, a.ubatch)
    if a.verbose:
        for w, (scored, nll) in enumerate(r.windows):
            print(f"chunk {w + 1}: scored {scored}, mean NLL {nll / scored:.9f}")
    print(f"tokens: {len(ids)}")
    print(f"used tokens: {r.used_tokens}")
    print(f"scored tokens: {r.scored_tokens}")
    print(f"chunks: {len(r.windows)}")
    print(f"context size: {r.context}")
    print(f"mean NLL: {r.mean_nll:.9f}")
    print(f"perplexity: {r.perplexity:.6g}")
    return 0


def cmd_replay(a) -> int:
    from .tools.trace_run import main as replay
    return replay(a.rest)


def cmd_bench(rest) -> int:
    """With --model (or --config and --random): the reference's model bench, cmd_bench_model.  Otherwise bench.py at
    the repository's root, with its own flags: the decode and prefill record at the real layer sizes."""
    if any(w == "--model" or w.startswith("--model=") or w == "--config" or w.startswith("--config=") for w in rest):
        return cmd_bench_model(list(rest))
    import runpy
    script = Path(__file__).resolve().parent.parent / "bench.py"
    old = sys.argv
    sys.argv = [str(script)] + list(rest)
    try:
        runpy.run_path(str(script), run_name="__main__")
    except SystemExit as e:
        return int(e.code or 0)
    finally:
        sys.argv = old
    return 0


def bench_model_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="llmx bench", description="prompt and decode rates of a model (the reference's `bench --model`)")
    ap.add_argument("--model", default=None, action=_Once, help="a model folder")
    ap.add_argument("--p", type=int, default=64, action=_Once, help="prompt tokens (default %(default)s)")
    ap.add_argument("--n", type=int, default=64, action=_Once, help="decoded tokens (default %(default)s)")
    ap.add_argument("--r", type=int, default=3, action=_Once, help="timed repetitions of each test (default %(default)s)")
    ap.add_argument("--seqs", type=int, default=1, action=_Once, help="sequences decoding together (default %(default)s)")
    ap.add_argument("--depth", type=int, default=0, action=_Once, help="tokens of history each test runs after; one sequence only (default %(default)s)")
    _add_exec(ap)
    return ap


def cmd_bench_model(argv) -> int:
    """`llmx bench --model DIR [--p 64] [--n 64] [--r 3] [--seqs 1] [--depth 0]`, the reference's model bench
    (/root/reference/src/cli/main.cpp:67-75,1192-1287): the rate of a prompt of p tokens after `depth` tokens of
    history, and of n decoded tokens (one sequence after the history; or `seqs` sequences together, each after the
    prompt, with each step's logits read on the host as a server would), as mean and standard deviation over r runs
    after one run that is not counted.  `--config JSON --random SEED` stands for the folder as elsewhere."""
    import statistics
    import torch
    from .engine import StepEntry
    a = bench_model_parser().parse_args(argv)
    a.words = [a.model] if a.model is not None else []
    _model_and_prompt(a, "bench")
    for name in ("p", "n", "r", "seqs"):
        if getattr(a, name) < 1:
            raise SystemExit2(f"bench: --{name} must be at least 1")
    if a.depth < 0 or (a.depth and a.seqs > 1):
        raise SystemExit2("bench: --depth is at least 0 and goes with one sequence")
    cfg = _config_of(a)
    P, G, R, S, D = a.p, a.n, a.r, a.seqs, a.depth
    reach = P + G if S > 1 else D + max(P, G)
    pages = -(-reach // a.page_tokens) + 1
    engine = _engine(a, cfg, kv_tokens=a.kv_tokens or S * pages * a.page_tokens, page_tokens=a.page_tokens, max_requests=S)
    vocab = cfg.vocab_size
    prompt, gen, history = _lcg_ids(P, vocab, 12345), _lcg_ids(G, vocab, 777), _lcg_ids(D, vocab, 4242)

    def feed(request, ids, want_last):
        for s in range(0, len(ids), a.ubatch):
            part = ids[s:s + a.ubatch]
            last = s + a.ubatch >= len(ids)
            engine.step([StepEntry(request, part, [len(part) - 1] if want_last and last else [])])

    def fresh(request):
        engine.add_request(request)
        if D:
            feed(request, history, False)
        torch.cuda.synchronize()

    def timed(work, tokens):
        t0 = time.perf_counter()
        work()
        torch.cuda.synchronize()
        return tokens / (time.perf_counter() - t0)

    def pp():
        fresh(0)
        rate = timed(lambda: feed(0, prompt, True), P)
        engine.end_request(0)
        return rate

    def tg():
        if S == 1:
            fresh(0)
            rate = timed(lambda: [engine.step([StepEntry(0, [t], [0])]) for t in gen], G)
            engine.end_request(0)
            return rate
        for q in range(S):
            engine.add_request(q)
            feed(q, prompt, True)
        torch.cuda.synchronize()
        rate = timed(lambda: [engine.step([StepEntry(q, [t], [0]) for q in range(S)]).cpu() for t in gen], G * S)
        for q in range(S):
            engine.end_request(q)
        return rate

    def report(what, n, rates):
        sd = statistics.stdev(rates) if len(rates) > 1 else 0.0
        at = f" @ d{D}" if D else ""
        print(f"bench: {what}{n}{at}  {statistics.mean(rates):8.2f} +- {sd:.2f} tok/s  ({len(rates)} runs)")

    pp()
    tg()
    report("pp", P, [pp() for _ in range(R)])
    report(f"x{S} tg" if S > 1 else "tg", G, [tg() for _ in range(R)])
    return 0


def cmd_random(a) -> int:
    """Writes a model folder (config.json, model.safetensors) with seeded random weights."""
    from .models import read_config
    from .weights import RandomInit
    from .weights.folder import write_random_model
    cfg = read_config(json.loads(Path(a.config).read_text()))
    write_random_model(a.out, cfg, RandomInit(seed=a.seed, std=a.std, norm_std=a.norm_std, bias_range=a.bias_range, storage=a.storage))
    print(a.out)
    return 0


def build_parser():
    ap = argparse.ArgumentParser(prog="llmx", description="MiniMax-M3 on one MI355X: generate, logits, perplexity, replay, random, bench")
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="generate tokens after a prompt of token ids")
    g.add_argument("words", nargs="*", metavar="MODEL [PROMPT]",
                   help="model folder (config.json + model.safetensors), then token ids, comma or space separated; with --config the prompt alone")
    g.add_argument("--file", "-f", default=None, help="a file with one prompt of token ids per line")
    g.add_argument("--prompt-len", type=int, default=0, help="make up a prompt of this many fixed token ids")
    _add_sampling(g)
    _add_exec(g)
    g.set_defaults(run=cmd_generate)
    l = sub.add_parser("logits", help="top logits of the last positions of a prompt")
    l.add_argument("words", nargs="*", metavar="MODEL [PROMPT]")
    l.add_argument("--file", "-f", default=None)
    l.add_argument("--then-ids", default=None, help="a file of token ids appended to the prompt")
    l.add_argument("--last", type=int, default=0, help="report this many final positions")
    l.add_argument("--per-token", action="store_true", help="feed the tokens one step each")
    l.add_argument("--top", type=int, default=10)
    _add_exec(l)
    l.set_defaults(run=cmd_logits)
    x = sub.add_parser("perplexity", help="mean negative log-likelihood of token ids, in windows from an empty history")
    x.add_argument("words", nargs="*", metavar="MODEL [PROMPT]")
    x.add_argument("--file", "-f", default=None, help="a file of token ids")
    x.add_argument("--ctx-size", "-c", type=int, default=0, action=_Once, help="window tokens (default: all the ids, at most the model's context)")
    x.add_argument("--chunks", type=int, default=0, action=_Once, help="windows at most (default: all)")
    x.add_argument("--per-token", action="store_true", help="one token a step: the decode path")
    _add_exec(x)
    x.set_defaults(run=cmd_perplexity)
    t = sub.add_parser("replay", help="feed a trace of steps through the model and write logits (bin/trace_run)", add_help=False)
    t.add_argument("rest", nargs=argparse.REMAINDER)
    t.set_defaults(run=cmd_replay)
    r = sub.add_parser("random", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--norm-std", type=float, default=0.0)
    r.add_argument("--bias-range", type=float, default=0.0)
    r.add_argument("--storage", choices=["bfloat16", "float32"], default="bfloat16")
    r.set_defaults(run=cmd_random)
    b = sub.add_parser("bench", help="--model DIR --p --n --r --seqs --depth: prompt and decode rates of a model; without a model: bench.py's record")
    b.add_argument("rest", nargs=argparse.REMAINDER)
    b.set_defaults(run=lambda a: cmd_bench(a.rest))
    return ap


def main(argv=None) -> int:
    ap = build_parser()
    argv = sys.argv[1:] if argv is None else list(argv)
    try:
        if argv and argv[0] == "replay":      # its own parser reads every flag, --help included
            return cmd_replay(argparse.Namespace(rest=argv[1:]))
        if argv and argv[0] == "bench":
            return cmd_bench(argv[1:])
        a = ap.parse_args(argv)
        return a.run(a)
    except SystemExit2 as e:
        print(f"llmx: {e}", file=sys.stderr)
        return 2
    except ValueError as e:
        # configuration, weights, sampling and scheduling refusals carry their own text
        print(f"llmx: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
