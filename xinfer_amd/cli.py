"""Command line in the reference's manner: option names and meanings of its `Args`
(/root/reference/src/server/mod.rs:706-904) and of its Python twin
(/root/reference/example/completion.py), for the options whose parts exist here.

    python -m xinfer_amd --m /path/to/model --prompts "How are you?|Tell me a story" --max-tokens 64
    python -m xinfer_amd --w /path/to/model --batch 8 --max-tokens 128 --temperature 0

Output per prompt and the two throughput lines follow /root/reference/src/main.rs:541-555.
"""
from __future__ import annotations

import argparse
import sys
import warnings
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="xinfer_amd", description="xinfer_amd command line")
    p.add_argument("--m", type=str, default=None, help="model folder (config.json, model.safetensors)")
    p.add_argument("--w", type=str, default=None, help="the same, under the legacy name")
    p.add_argument("--dtype", type=str, default="bf16", help="bf16 (default) or f32")
    p.add_argument("--prompts", type=str, default=None, help="use '|' to separate multiple prompts")
    p.add_argument("--prompt-ids", type=str, default=None,
                   help="prompts as token ids: '1,2,3|4,5' (for models without a tokenizer)")
    p.add_argument("--max-num-seqs", type=int, default=1, help="most concurrent sequences")
    p.add_argument("--max-model-len", type=int, default=None)
    p.add_argument("--max-tokens", type=int, default=16384, help="max tokens for each request")
    p.add_argument("--ignore-eos", action="store_true", help="continue after an EOS token")
    p.add_argument("--batch", type=int, default=None, help="repeat the first prompt N times (performance test)")
    p.add_argument("--temperature", type=float, default=None)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--top-p", type=float, default=None)
    p.add_argument("--frequency-penalty", type=float, default=None)
    p.add_argument("--presence-penalty", type=float, default=None)
    p.add_argument("--seed", type=int, default=None, help="seed to reproduce results")
    p.add_argument("--kv-fraction", type=float, default=None,
                   help="share of the GPU memory left after loading that the cache may take")
    p.add_argument("--prefill-chunk-size", type=int, default=8192,
                   help="most prompt tokens of one request in a step")
    p.add_argument("--disable-cuda-graph", action="store_true", help="disable HIP graph replay of decode steps")
    p.add_argument("--yarn-scaling-factor", type=float, default=None,
                   help="stretch the model's positions by this factor with YaRN")
    p.add_argument("--i", dest="interactive", action="store_true",
                   help="interactive chat: prompts are read line by line, the conversation so far is the context")
    p.add_argument("--page-size", type=int, default=64, help="tokens per cache page")
    p.add_argument("--num-pages", type=int, default=None, help="cache pages (default: from --kv-fraction)")
    return p


def run(args) -> int:
    from . import EngineConfig, GenerationConfig, SamplingParams
    from .engine.llm_engine import LLMEngine

    if args.m and args.w:
        print("Use either --m <model> or legacy --w <local_dir>, not both.", file=sys.stderr)
        return 2
    if not (args.m or args.w):
        print("Must provide model folder (--m or --w)!", file=sys.stderr)
        return 2
    interactive = bool(args.interactive)
    if interactive and args.batch:
        print("interactive mode is ignored in batch performance test.", file=sys.stderr)   # main.rs:58-60
        interactive = False
    if interactive:
        prompts: List = []
    elif args.prompt_ids:
        prompts = [[int(t) for t in part.split(",") if t.strip()] for part in args.prompt_ids.split("|")]
    elif args.prompts:
        prompts = args.prompts.split("|")
    else:
        prompts = ["How are you?", "How to make money?"]
        print("No prompts found, use default ", prompts)
    if args.batch and args.batch > 1:
        prompts = [prompts[0]] * args.batch              # main.rs:103-115
    max_num_seqs = max(args.max_num_seqs, len(prompts))
    max_model_len = args.max_model_len
    if max_model_len is None:
        max_model_len = 32768 // max_num_seqs            # completion.py:34-38
        warnings.warn(f"max_model_len is not given, default to {max_model_len}.")
    gen_cfg = None
    if (args.temperature is not None and (args.top_p is not None or args.top_k is not None)) \
            or args.frequency_penalty is not None or args.presence_penalty is not None:
        gen_cfg = GenerationConfig(args.temperature, args.top_p, args.top_k,
                                   args.frequency_penalty, args.presence_penalty)
    cfg = EngineConfig(
        model_id=args.m, weight_path=args.w, max_num_seqs=max_num_seqs, max_model_len=max_model_len,
        max_tokens=min(args.max_tokens, max_model_len), generation_cfg=gen_cfg, seed=args.seed,
        kv_fraction=args.kv_fraction, prefill_chunk_size=args.prefill_chunk_size,
        disable_cuda_graph=args.disable_cuda_graph, page_size=args.page_size, num_pages=args.num_pages,
        yarn_scaling_factor=args.yarn_scaling_factor)
    engine = LLMEngine(cfg, args.dtype)
    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            frequency_penalty=args.frequency_penalty,
                            presence_penalty=args.presence_penalty, ignore_eos=args.ignore_eos)
    if interactive:
        return _chat(engine, params, max_num_seqs * max_model_len)
    print("Start inference with", len(prompts), "prompts")
    outputs = engine.generate(prompts, [params] * len(prompts))
    outputs.sort(key=lambda o: o.seq_id)
    prompt_time = decode_time = 0.0
    total_prompt = total_decoded = 0
    for i, o in enumerate(outputs):
        if not (args.batch and args.batch > 1):
            print(f"\n[Prompt {i + 1}]")
            print(f"Prompt: {prompts[i]}")
            print(f"Response: {o.decode_output}")
        total_prompt += o.prompt_length
        total_decoded += o.decoded_length
        prompt_time = max(prompt_time, (o.decode_start_time - o.prompt_start_time) / 1000.0)
        decode_time = max(decode_time, (o.decode_finish_time - o.decode_start_time) / 1000.0)
    print("\n--- Performance Metrics ---")
    print(f"Prompt tokens: {total_prompt} in {prompt_time:.2f}s "
          f"({total_prompt / max(prompt_time, 0.001):.2f} tokens/s)")
    print(f"Decoded tokens: {total_decoded} in {decode_time:.2f}s "
          f"({total_decoded / max(decode_time, 0.001):.2f} tokens/s)")
    return 0


def _chat(engine, params, total_tokens: int, lines=None, out=None) -> int:
    """The reference's interactive mode (main.rs:320-560): every line is a user turn of one
    conversation whose history is the context; the answer is printed as its tokens arrive.  An
    empty line asks again; end of input (or Ctrl+C) clears the history if there is one and
    exits if there is none."""
    from . import Message
    out = out or sys.stdout
    lines = iter(lines) if lines is not None else None
    history: List = []
    left = total_tokens
    while True:
        print("Enter a new prompt (Press Ctrl+C to exit):" if not history else
              "Enter another prompt to continue current chat (Press Ctrl+C to start a new chat):", file=out, flush=True)
        try:
            line = next(lines) if lines is not None else input()
        except (EOFError, KeyboardInterrupt, StopIteration):
            if not history:
                print("Exiting.", file=out, flush=True)
                return 0
            print("Chat history cleared. Start a new conversation.", file=out, flush=True)
            history.clear()
            left = total_tokens
            continue
        text = line.strip()
        if not text:
            print("No prompt was given.", file=out, flush=True)
            continue
        if left <= 0:
            print("No tokens left, press Ctrl+C to start a new chat session!", file=out, flush=True)
            continue
        history.append(Message("user", text))
        try:
            seq_id, prompt_length, stream = engine.generate_stream(params, list(history))
        except Exception as ex:          # the conversation no longer fits: start over, as the reference does
            print(f"Session unexpectedly ended because: {ex}", file=out, flush=True)
            print("Chat history cleared. Start a new conversation.", file=out, flush=True)
            history.clear()
            left = total_tokens
            continue
        pieces: List[str] = []
        decoded = 0
        for item in stream:
            if item.datatype == "TOKEN":
                pieces.append(item.data)
                print(item.data, end="", file=out, flush=True)
            elif item.datatype == "TOKEN_ID":
                decoded += 1
            elif item.datatype == "ERROR":
                print(f"\n{item.data}", file=out, flush=True)
        print(file=out, flush=True)
        history.append(Message("assistant", "".join(pieces)))
        left = total_tokens - prompt_length - decoded
        print(f"Tokens left: {left}", file=out, flush=True)


def main(argv: Optional[List[str]] = None) -> int:
    return run(build_parser().parse_args(argv))
