"""LongBench and GSM8K runs with the polar-key models, as the reference's scripts make them
(test4long.py, test4gsm8k.py): build the prompt, cut over-long prompts in the middle, generate
greedily with the reference's decoding loop, score with the reference's metrics, write one JSON
line per example.  One process, one GPU (the reference spreads the examples over processes with
`accelerate`; the examples are independent, so the scores do not depend on that).

    python -m polarquant_amd.accuracy_eval longbench --model /path/to/llama-3.1-8b-instruct \\
        --data /path/to/longbench --out out/longbench [--datasets hotpotqa lcc] [--max-length 120000]
    python -m polarquant_amd.accuracy_eval gsm8k --model /path/to/llama-3.1-8b-instruct \\
        --data /path/to/gsm8k.json --out out/gsm8k.jsonl [--shots shots.txt]

`--data` for LongBench is a directory with `dataset2prompt.json`, `dataset2maxlen.json` and one
`<dataset>.jsonl` per task (LongBench's published files); for GSM8K a file with one JSON object per
line, `{"conversations": [{"value": question}, {"value": "... The answer is N"}]}`, the layout the
reference reads.  Neither data set, nor any checkpoint, ships with this package.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from . import eval_metrics as metrics
from .modeling_common import generate

LONGBENCH_DATASETS = ("narrativeqa", "qasper", "multifieldqa_en", "2wikimqa", "hotpotqa", "musique", "lcc", "repobench-p")
CODE_DATASETS = ("lcc", "repobench-p")          # completed as plain text, without a chat template (test4long.py:110)

# single-turn chat formats of the model families the reference evaluates (test4long.py:110-121)
CHAT_TEMPLATES = {
    "llama3": "<|start_header_id|>user<|end_header_id|>\n\n{prompt}<|eot_id|><|start_header_id|>assistant<|end_header_id|>\n\n",
    "llama2": "[INST]{prompt}[/INST]",
    "qwen2": "<|im_start|>user\n{prompt}<|im_end|>\n<|im_start|>assistant\n",
    "none": "{prompt}",
}
# turn formats of the GSM8K few-shot dialogue (test4gsm8k.py:113-117): (question turn, answer turn, answer opener)
GSM8K_TURNS = {
    "llama3": ("<|start_header_id|>user<|end_header_id|>\n\n{query}<|eot_id|>",
               "<|start_header_id|>assistant<|end_header_id|>\n\n{reply}<|eot_id|>",
               "<|start_header_id|>assistant<|end_header_id|>\n\n"),
    "none": ("{query}\n", "{reply}\n\n", ""),
}
THINK = "Let's think step by step\n"

# Worked examples for the few-shot prompt when no --shots file is given.  They are this package's own; the
# reference's script carries eight of its own in the same layout, and its published accuracy was made with those.
DEFAULT_SHOTS = """Question: A box holds 6 rows of 7 pencils. How many pencils are in 3 boxes?
Let's think step by step
One box holds 6*7=42 pencils.
Three boxes hold 42*3=126 pencils.
The answer is 126

Question: Mara had 50 dollars and bought 4 books for 9 dollars each. How many dollars does she have left?
Let's think step by step
The books cost 4*9=36 dollars.
She has 50-36=14 dollars left.
The answer is 14

Question: A train covers 240 km in 4 hours. How many km does it cover in 7 hours at the same speed?
Let's think step by step
Its speed is 240/4=60 km per hour.
In 7 hours it covers 60*7=420 km.
The answer is 420

Question: Half of a number, less 5, is 11. What is the number?
Let's think step by step
Half of the number is 11+5=16.
The number is 16*2=32.
The answer is 32"""


def truncate_middle(ids: Sequence[int], max_length: int) -> List[int]:
    """A prompt longer than `max_length` tokens keeps its first and last max_length // 2 tokens (test4long.py:134-135)."""
    ids = list(ids)
    if len(ids) <= max_length:
        return ids
    half = max_length // 2
    return ids[:half] + ids[-half:]


def longbench_prompt(template: str, example: Dict, dataset: str, chat: str) -> str:
    prompt = template.format(**example)
    return prompt if dataset in CODE_DATASETS else CHAT_TEMPLATES[chat].format(prompt=prompt)


def gsm8k_prefix(shots_text: str, chat: str) -> str:
    """The few-shot dialogue in front of every question: each worked example as a question turn and an answer turn."""
    q_turn, a_turn, _ = GSM8K_TURNS[chat]
    out = ""
    for block in shots_text.strip().split("\n\n"):
        body = block.split("Question: ", 1)[1]
        query, _, reply = body.partition("\n")
        out += q_turn.format(query=query) + a_turn.format(reply=reply)
    return out


def gsm8k_prompt(prefix: str, question: str, chat: str) -> str:
    q_turn, _, opener = GSM8K_TURNS[chat]
    return prefix + q_turn.format(query=question) + opener + THINK


def complete(model, tokenizer, generation_config, input_ids: Sequence[int], max_new_tokens: int, graph_decoder: bool = False) -> str:
    """Greedy continuation of one prompt, decoded without special tokens (test4long.py:137-139)."""
    ids = torch.tensor([list(input_ids)], device=model.device)
    out = generate(model, input_ids=ids, attention_mask=None, max_new_tokens=max_new_tokens,
                   generation_config=generation_config, graph_decoder=graph_decoder)
    return tokenizer.batch_decode(out, skip_special_tokens=True)[0]


def _read_jsonl(path: str, limit: Optional[int]) -> List[Dict]:
    rows = []
    with open(path) as f:
        for line in f:
            if line.strip():
                rows.append(json.loads(line))
                if limit is not None and len(rows) >= limit:
                    break
    return rows


def _write_jsonl(path: str, rows: Iterable[Dict]) -> None:
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        for r in rows:
            f.write(json.dumps(r) + "\n")


def run_longbench(model, tokenizer, generation_config, data_dir: str, out_dir: str,
                  datasets: Sequence[str] = LONGBENCH_DATASETS, max_length: int = 120000, chat: str = "llama3",
                  limit: Optional[int] = None, graph_decoder: bool = False,
                  progress: Optional[Callable[[str], None]] = None) -> Dict[str, float]:
    """-> {dataset: mean score in [0, 1]}; writes `<out_dir>/<dataset>.jsonl` (idx, output_text, answers, score)."""
    with open(os.path.join(data_dir, "dataset2prompt.json")) as f:
        templates = json.load(f)
    with open(os.path.join(data_dir, "dataset2maxlen.json")) as f:
        new_tokens = json.load(f)
    results = {}
    for dataset in datasets:
        metric = metrics.LONGBENCH_METRIC[dataset]
        rows = []
        for idx, ex in enumerate(_read_jsonl(os.path.join(data_dir, dataset + ".jsonl"), limit)):
            ids = truncate_middle(tokenizer.encode(longbench_prompt(templates[dataset], ex, dataset, chat)), max_length)
            text = complete(model, tokenizer, generation_config, ids, int(new_tokens[dataset]), graph_decoder)
            score = metrics.best_score(metric, text, ex["answers"], ex.get("all_classes"))
            rows.append({"idx": idx, "output_text": text, "answers": ex["answers"], "score": score})
            if progress:
                progress("%s %d: %d prompt tokens, score %.3f" % (dataset, idx, len(ids), score))
        _write_jsonl(os.path.join(out_dir, dataset + ".jsonl"), rows)
        results[dataset] = sum(r["score"] for r in rows) / len(rows) if rows else 0.0
        if progress:
            progress("%s: %d examples, score %.2f" % (dataset, len(rows), 100 * results[dataset]))
    return results


def run_gsm8k(model, tokenizer, generation_config, test_file: str, out_file: str, shots_text: str = DEFAULT_SHOTS,
              chat: str = "llama3", limit: Optional[int] = None, max_new_tokens: int = 256, graph_decoder: bool = False,
              progress: Optional[Callable[[str], None]] = None) -> float:
    """-> accuracy in [0, 1]; writes `out_file` (idx, output_text, answers, score).  The generated text is cut at
    its first blank line before it is judged (test4gsm8k.py:171)."""
    prefix = gsm8k_prefix(shots_text, chat)
    rows = []
    for idx, ex in enumerate(_read_jsonl(test_file, limit)):
        question, answer = ex["conversations"][0]["value"], ex["conversations"][1]["value"]
        ids = tokenizer.encode(gsm8k_prompt(prefix, question, chat))
        text = complete(model, tokenizer, generation_config, ids, max_new_tokens, graph_decoder).split("\n\n")[0]
        score = metrics.judge_gsm8k(text, answer)
        rows.append({"idx": idx, "output_text": text, "answers": answer, "score": score})
        if progress:
            progress("gsm8k %d: %s" % (idx, "right" if score else "wrong"))
    _write_jsonl(out_file, rows)
    return sum(r["score"] for r in rows) / len(rows) if rows else 0.0


def _load(args) -> Tuple:
    from transformers import AutoTokenizer
    from .checkpoint import load_generation_config, load_pretrained
    tokenizer = AutoTokenizer.from_pretrained(args.model, use_fast=True)
    options = dict(rbits=args.rbits, tbits=args.tbits, vbits=4 if args.variant == "mixed" else 16, snapkv=args.variant == "snapkv")
    model = load_pretrained(args.model, torch.bfloat16, "cuda:0", **options)
    return model, tokenizer, load_generation_config(args.model)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    sub = ap.add_subparsers(dest="task", required=True)
    for name in ("longbench", "gsm8k"):
        p = sub.add_parser(name)
        p.add_argument("--model", required=True, help="checkpoint directory (config.json, safetensors, tokenizer files)")
        p.add_argument("--data", required=True)
        p.add_argument("--out", required=True)
        p.add_argument("--variant", choices=("polar", "mixed", "snapkv"), default="polar",
                       help="polar keys; polar keys + 4-bit values; SnapKV prompt eviction in front of polar keys")
        p.add_argument("--rbits", type=int, default=4)
        p.add_argument("--tbits", type=int, default=4)
        p.add_argument("--limit", type=int, default=None, help="only the first N examples of each file")
        p.add_argument("--graph", action="store_true", help="replay the decode step from a captured HIP graph")
    sub.choices["longbench"].add_argument("--datasets", nargs="+", default=list(LONGBENCH_DATASETS), choices=LONGBENCH_DATASETS)
    sub.choices["longbench"].add_argument("--max-length", type=int, default=120000)
    sub.choices["longbench"].add_argument("--chat", choices=sorted(CHAT_TEMPLATES), default="llama3")
    sub.choices["gsm8k"].add_argument("--shots", default=None, help="text file of worked examples (Question: ... / The answer is N, blank line between)")
    sub.choices["gsm8k"].add_argument("--chat", choices=sorted(GSM8K_TURNS), default="llama3")
    args = ap.parse_args(argv)
    torch.manual_seed(42 if args.task == "longbench" else 0)
    model, tokenizer, gen = _load(args)
    say = lambda s: print(s, file=sys.stderr, flush=True)
    if args.task == "longbench":
        res = run_longbench(model, tokenizer, gen, args.data, args.out, args.datasets, args.max_length, args.chat,
                            args.limit, args.graph, say)
        print(json.dumps({"task": "longbench", "scores_x100": {k: round(100 * v, 2) for k, v in res.items()}}))
    else:
        shots = DEFAULT_SHOTS
        if args.shots:
            with open(args.shots) as f:
                shots = f.read()
        acc = run_gsm8k(model, tokenizer, gen, args.data, args.out, shots, args.chat, args.limit, graph_decoder=args.graph, progress=say)
        print(json.dumps({"task": "gsm8k", "accuracy_x100": round(100 * acc, 2)}))


if __name__ == "__main__":
    main()
