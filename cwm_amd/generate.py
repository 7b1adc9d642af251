"""Command line of the engine: token ids in, token ids out.

    python -m cwm_amd.generate checkpoint_dir=MODEL_DIR prompts=prompts.jsonl \\
        gen_args.max_batch=8 gen_args.max_seq=8192 gen_args.temperature=0.6 gen_args.top_p=0.95

Options are given as `key=value` and `group.key=value`, after an optional
`config=file.yaml`, as the reference's server takes them
(`python -m serve.fgserve config=... checkpoint_dir=... gen_args.x=y`,
serve/README.md:7-9; option record serve/fgserve.py:68-83).  `gen_args.*` are the
reference's generation options (cwm/fastgen/generate.py:37-68).  The server part of
the reference (HTTP, chat formats, tokenizer) is not built: requests are lines of
JSON, {"id": ..., "tokens": [...], "max_gen": ..., "temperature": ..., "top_p": ...},
read from the file `prompts` (`-` for standard input) or given inline with
`prompt=[1,2,3]`; each result is printed as one line of JSON,
{"id": ..., "tokens": [...], "finish_reason": ...}, as the reference's
/completions answers with "tokens" (serve/fgserve.py:266-274).
"""

from __future__ import annotations

import json
import logging
import queue
import sys
import time
from dataclasses import dataclass, field
from typing import List, Optional

from .config.cli import load_from_cli
from .config.schema import ConfigError
from .engine.api import GenArgs, Packet


@dataclass
class ServeGenArgs(GenArgs):
    """The reference's server defaults (serve/fgserve.py:54-66)."""

    use_sampling: bool = True
    temperature: float = 0.6
    top_p: float = 0.95
    max_batch: int = 256
    sync_freq: int = 1


@dataclass
class GenerateArgs:
    checkpoint_dir: str = ""  # folder with config.json and *.safetensors
    gen_args: ServeGenArgs = field(default_factory=ServeGenArgs)
    seed: int = 17
    log_level: str = "info"
    perf_log_freq: int = 60  # seconds between throughput lines on stderr

    prompts: str = ""  # JSON-lines file of requests, "-" for standard input
    prompt: Optional[List[int]] = None  # one request given inline
    out: str = ""  # file for the results (default: standard output)
    dtype: str = "bfloat16"  # bfloat16 | float32
    device: str = "cuda:0"
    stop_tokens: List[int] = field(default_factory=list)  # ids that end a request (kept as its last token)
    random_config: str = ""  # a config.json to run with random weights instead of checkpoint_dir
    weight_seed: int = 0  # seed of those random weights


def _read_requests(args: GenerateArgs) -> List[Packet]:
    packets: List[Packet] = []
    if args.prompt is not None:
        packets.append(Packet(thread_id=0, tokens=list(args.prompt)))
    if args.prompts:
        fh = sys.stdin if args.prompts == "-" else open(args.prompts, "r", encoding="utf-8")
        try:
            for line in fh:
                line = line.strip()
                if not line:
                    continue
                rec = json.loads(line)
                packets.append(
                    Packet(
                        thread_id=rec.get("id", len(packets)),
                        tokens=[int(t) for t in rec["tokens"]],
                        max_gen=rec.get("max_gen"),
                        temperature=rec.get("temperature"),
                        top_p=rec.get("top_p"),
                        seed=rec.get("seed"),
                    )
                )
        finally:
            if fh is not sys.stdin:
                fh.close()
    if not packets:
        raise ConfigError("no request given: use prompts=FILE, prompts=- or prompt=[ids]")
    return packets


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if any(a in ("-h", "--help") for a in argv):
        print(__doc__)
        return 0
    try:
        args = load_from_cli(GenerateArgs, argv)
    except ConfigError as exc:
        print(f"error: {exc}", file=sys.stderr)
        return 2
    logging.basicConfig(level=getattr(logging, args.log_level.upper(), logging.INFO), stream=sys.stderr,
                        format="%(asctime)s %(levelname)s %(message)s")
    log = logging.getLogger("cwm_amd")

    from .engine.engine import Engine

    if bool(args.checkpoint_dir) == bool(args.random_config):
        print("error: give exactly one of checkpoint_dir=DIR and random_config=FILE", file=sys.stderr)
        return 2
    packets = _read_requests(args)
    if args.random_config:
        with open(args.random_config, "r", encoding="utf-8") as fh:
            config = json.load(fh)
        engine = Engine.from_random(config, args.weight_seed, args.gen_args, args.dtype, args.device, args.stop_tokens, args.seed)
    else:
        engine = Engine.from_folder(args.checkpoint_dir, args.gen_args, args.dtype, args.device, args.stop_tokens, args.seed)
    engine.install_profile_signal()  # kill -USR2 PID traces a window of steps (FG_PROFILE_ITERS, FG_PROFILE_DIR)
    log.info("cache: %d tokens in pages of %d; max_batch %d", engine.max_seq, args.gen_args.cache_block, args.gen_args.max_batch)

    q: "queue.Queue[Optional[Packet]]" = queue.Queue()
    for packet in packets:
        q.put(packet)
    q.put(None)
    out = open(args.out, "w", encoding="utf-8") if args.out else sys.stdout
    last = time.time()
    steps = seqs = toks = 0
    try:
        for packet in engine.generate(q):
            now = time.time()
            if now - last > args.perf_log_freq:
                # serve/fgserve.py:330-349
                dt = now - last
                log.info(
                    "Generation performance: %.2f calls/s, %.2f seqs/s, %.1f toks/s",
                    (engine.n_steps - steps) / dt, (engine.n_sequences - seqs) / dt, (engine.n_generated - toks) / dt,
                )
                last, steps, seqs, toks = now, engine.n_steps, engine.n_sequences, engine.n_generated
            if packet is None:
                continue
            rec = {"id": packet.thread_id, "tokens": packet.tokens, "finish_reason": packet.finish_reason}
            if packet.logprobs is not None:
                rec["logprobs"] = packet.logprobs
                rec["sample_logprobs"] = packet.sample_logprobs
            print(json.dumps(rec), file=out, flush=True)
    finally:
        if out is not sys.stdout:
            out.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
