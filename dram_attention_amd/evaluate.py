"""Key-value recall harness around the Llama-shaped model.

Counterpart of the reference's evaluation driver
(evaluation/dram-attention/evaluate.py:47-178 and read_eval_result.py:1-44; the
same files exist for the comparison models under evaluation/quest,
evaluation/quest-top-k-oracle and evaluation/full-attention): load a Llama-3
checkpoint directory (``params.json``, ``consolidated.00.pth``,
``tokenizer.model``), feed every item of a RULER ``niah_multikey_2``
``validation_<seq_len>.jsonl`` file as page-aligned prefill + token-by-token
decode, take the first number of the completion as the answer, write one JSON
line per item and report the average recall per sequence length.

    python -m dram_attention_amd.evaluate --model-dir … --data-dir … --seq-len 8192
    python -m dram_attention_amd.evaluate --report          # table over eval_results_*.jsonl

Differences from the reference's script: ``--top-k``, ``--page-size`` and
``--local-attn-window`` reach the model (the reference logs them but builds its
``ModelArgs`` from the defaults, evaluate.py:51-55); ``--variant`` picks which
of the four evaluated models the attention layers form; ``--tokenizer bytes``
and ``--synthetic N`` run the harness without the tiktoken vocabulary and
without the RULER files (plumbing only: recall needs the trained weights).
Neither the weights nor the data are part of this repository.
"""
from __future__ import annotations

import argparse
import glob
import json
import logging
import os
import re
from pathlib import Path
from typing import Iterable, Iterator, List, Optional, Sequence

import torch

from .llama import ModelArgs, Transformer

logger = logging.getLogger(__name__)

PARAMS_KEYS = ("dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "multiple_of",
               "ffn_dim_multiplier", "norm_eps", "rope_theta", "use_scaled_rope")


def load_model(ckpt_dir: str, max_seq_len: int, *, variant: str = "dram", top_k: int = 4096,
               page_size: int = 16, local_attn_window: int = 4096, local_margin: int = 1024,
               lru_hbm_cache_size: int = 32 * 1024, max_output_length: int = 128,
               dtype: torch.dtype = torch.bfloat16, device="cuda") -> Transformer:
    """``params.json`` + ``consolidated.00.pth`` -> model (evaluate.py:47-72).  The
    local cache is the attention window plus ``local_margin`` rows, as in the
    reference's default (4096 + 1024, model.py:41): room for the prompt tokens behind
    the page-aligned prefill and for the completion."""
    with open(Path(ckpt_dir) / "params.json") as f:
        params = json.load(f)
    unknown = sorted(set(params) - set(PARAMS_KEYS))
    if unknown:
        raise ValueError(f"params.json: unknown fields {unknown}")
    assert local_attn_window % page_size == 0 and top_k % page_size == 0
    args = ModelArgs(max_seq_len=max_seq_len, max_batch_size=1, cache_top_k=top_k,
                     cache_page_size=page_size, local_cache_size=local_attn_window + local_margin,
                     lru_hbm_cache_size=lru_hbm_cache_size, max_output_length=max_output_length,
                     attention_variant=variant, dtype=dtype, **params)
    model = Transformer(args, device=device)
    state = torch.load(Path(ckpt_dir) / "consolidated.00.pth", map_location="cpu", mmap=True,
                       weights_only=True)
    # A checkpoint holds the weights; the caches are buffers of the model and start empty.
    # Rope tables of older checkpoints are recomputed, as with the reference's strict=False.
    weights = {name for name, _ in model.named_parameters()}
    missing = sorted(weights - set(state))
    unknown = sorted(k for k in set(state) - weights if not k.endswith("freqs"))
    if missing or unknown:
        raise KeyError(f"checkpoint lacks {missing[:4]} and has unknown tensors {unknown[:4]}")
    model.load_state_dict({k: state[k] for k in weights}, strict=False)
    logger.info("Model loaded from %s", ckpt_dir)
    return model


class ByteTokenizer:
    """UTF-8 bytes as tokens, for running the harness without a trained vocabulary:
    ids 0-255 are the bytes, then bos, eos, pad."""

    n_words = 259
    bos_id, eos_id, pad_id = 256, 257, 258
    special_start = 256

    @property
    def stop_tokens(self):
        return {self.eos_id}

    def encode(self, s: str, *, bos: bool, eos: bool) -> List[int]:
        return ([self.bos_id] if bos else []) + list(s.encode("utf-8")) + ([self.eos_id] if eos else [])

    def decode(self, ids: Sequence[int]) -> str:
        return bytes(i for i in ids if i < 256).decode("utf-8", errors="replace")


class TiktokenTokenizer:
    """The Llama-3 vocabulary file through ``tiktoken`` (evaluation/dram-attention/
    tokenizer.py:38-118): 256 special tokens after the merges, ``<|begin_of_text|>``
    first, pad = -1."""

    special_start = 128000
    pattern = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*"
               r"|\s*[\r\n]+|\s+(?!\S)|\s+")

    def __init__(self, model_path: str):
        try:
            import tiktoken
            from tiktoken.load import load_tiktoken_bpe
        except ImportError as e:  # pragma: no cover - the package is optional
            raise RuntimeError("the Llama-3 tokenizer needs the tiktoken package "
                               "(or run with --tokenizer bytes)") from e
        ranks = load_tiktoken_bpe(model_path)
        names = ["<|begin_of_text|>", "<|end_of_text|>", "<|reserved_special_token_0|>",
                 "<|reserved_special_token_1|>", "<|finetune_right_pad_id|>", "<|step_id|>",
                 "<|start_header_id|>", "<|end_header_id|>", "<|eom_id|>", "<|eot_id|>",
                 "<|python_tag|>"]
        names += [f"<|reserved_special_token_{2 + i}|>" for i in range(256 - len(names))]
        self.special_tokens = {n: len(ranks) + i for i, n in enumerate(names)}
        self.model = tiktoken.Encoding(name=Path(model_path).name, pat_str=self.pattern,
                                       mergeable_ranks=ranks, special_tokens=self.special_tokens)
        self.n_words = len(ranks) + len(names)
        self.bos_id = self.special_tokens["<|begin_of_text|>"]
        self.eos_id = self.special_tokens["<|end_of_text|>"]
        self.pad_id = -1
        self.stop_tokens = {self.eos_id, self.special_tokens["<|eom_id|>"],
                            self.special_tokens["<|eot_id|>"]}

    def encode(self, s: str, *, bos: bool, eos: bool) -> List[int]:
        ids = self.model.encode(s, allowed_special=set(), disallowed_special=())
        return ([self.bos_id] if bos else []) + ids + ([self.eos_id] if eos else [])

    def decode(self, ids: Sequence[int]) -> str:
        return self.model.decode(list(ids))


@torch.inference_mode()
def generate(model: Transformer, prefix_prompt_tokens: Sequence[int],
             suffix_prompt_tokens: Sequence[int], max_gen_len: int, *, page_size: int,
             stop_tokens: Iterable[int], special_start: int) -> List[int]:
    """Greedy completion of prefix + suffix (evaluate.py:75-121).  The prefix, cut
    to whole pages, is one prefill call; every later position is a decode step
    that is fed the prompt token while there is one and the model's own choice
    afterwards.  Stops at a stop token, at any token of the special range, or at
    the length limit; returns the generated tokens ahead of that position."""
    dev = model.tok_embeddings.weight.device
    params = model.params
    prompt = list(prefix_prompt_tokens) + list(suffix_prompt_tokens)
    prompt_len = len(prompt)
    assert prompt_len <= params.max_seq_len
    total_len = min(params.max_seq_len, max_gen_len + prompt_len)
    aligned = len(prefix_prompt_tokens) // page_size * page_size
    assert 0 < aligned < total_len, "the prefix must hold at least one page"
    stop = set(stop_tokens)
    tokens = prompt + [0] * (total_len - prompt_len)

    def pick(logits, pos):  # position `pos` gets the prompt's token or the model's
        return tokens[pos] if pos < prompt_len else int(logits[0, -1].argmax().item())

    ids = torch.tensor([tokens[:aligned]], dtype=torch.long, device=dev)
    tokens[aligned] = pick(model(ids, 0), aligned)
    cur_pos = aligned
    for cur_pos in range(aligned, total_len - 1):
        step = torch.tensor([[tokens[cur_pos]]], dtype=torch.long, device=dev)
        nxt = pick(model(step, cur_pos), cur_pos + 1)
        tokens[cur_pos + 1] = nxt
        if nxt in stop or nxt >= special_start:
            break
    return tokens[prompt_len: cur_pos + 1]


def first_number(text: str) -> Optional[str]:
    """The answer the harness scores: the first run of digits (evaluate.py:157-158)."""
    m = re.search(r"\d+", text)
    return m.group() if m else None


def read_jsonl(path: str) -> Iterator[dict]:
    with open(path) as f:
        for line in f:
            if line.strip():
                yield json.loads(line)


def synthetic_niah(n_items: int, n_pairs: int, seed: int) -> List[dict]:
    """Items shaped like RULER's niah_multikey_2 records (``index``, ``input`` whose
    last line is the question, ``query``, ``answer`` list): key-value lines with
    two-word keys and 7-digit values, one of them asked for."""
    import random

    rng = random.Random(seed)
    words = ["amber", "birch", "cedar", "delta", "ember", "fjord", "grove", "heron", "inlet",
             "jetty", "knoll", "larch", "marsh", "north", "oasis", "prism", "quill", "ridge"]
    items = []
    for index in range(n_items):
        keys = set()
        while len(keys) < n_pairs:
            keys.add(f"{rng.choice(words)}-{rng.choice(words)}-{len(keys)}")
        pairs = [(k, str(rng.randrange(10 ** 6, 10 ** 7))) for k in sorted(keys)]
        rng.shuffle(pairs)
        key, value = pairs[rng.randrange(n_pairs)]
        body = "\n".join(f"One of the special magic numbers for {k} is: {v}." for k, v in pairs)
        question = f"What is the special magic number for {key} mentioned in the provided text? The number is"
        items.append({"index": index, "input": body + "\n" + question, "query": key,
                      "answer": [value]})
    return items


def evaluate_items(model: Transformer, tokenizer, items: Iterable[dict], *, page_size: int,
                   results_path: Optional[str] = None, max_gen_len: int = 32) -> float:
    """Runs every item and returns the average recall (evaluate.py:133-178): the
    lines before the last are the prefix (with bos), the last line the suffix."""
    total_recall = total_items = 0
    out = open(results_path, "w") if results_path else None
    try:
        for item in items:
            lines = item["input"].split("\n")
            prefix = tokenizer.encode("\n".join(lines[:-1]) + "\n", bos=True, eos=False)
            suffix = tokenizer.encode(lines[-1], bos=False, eos=False)
            logger.info("==== #%s ==== prompt length %d", item["index"], len(prefix) + len(suffix))
            got = generate(model, prefix, suffix, max_gen_len, page_size=page_size,
                           stop_tokens=tokenizer.stop_tokens, special_start=tokenizer.special_start)
            model_output = first_number(tokenizer.decode(got))
            recall = 1 if model_output is not None and model_output in item["answer"] else 0
            total_recall += recall
            total_items += 1
            result = {"index": item["index"], "query": item["query"], "answer": item["answer"],
                      "model_output": model_output, "recall": recall}
            logger.info("Result: %s", json.dumps(result))
            if out:
                out.write(json.dumps(result) + "\n")
                out.flush()
    finally:
        if out:
            out.close()
    return total_recall / total_items if total_items else 0.0


def average_recall(path: str) -> float:
    """Mean of the ``recall`` fields of a results file; lines that are not JSON or
    carry no recall are skipped (read_eval_result.py:5-25)."""
    total = n = 0
    with open(path) as f:
        for line in f:
            try:
                recall = json.loads(line).get("recall")
            except json.JSONDecodeError:
                continue
            if recall is not None:
                total += recall
                n += 1
    return total / n if n else 0.0


def report(directory: str = ".") -> str:
    """The table of read_eval_result.py:28-44 over ``eval_results_<seq_len>[_run].jsonl``."""
    rows = []
    for path in glob.glob(os.path.join(directory, "eval_results_*.jsonl")):
        seq_len = os.path.basename(path).split("_")[2].split(".")[0]
        rows.append((int(seq_len), f"{average_recall(path):.4f}"))
    rows.sort()
    lines = ["Sequence Length | Average Recall", "-" * 16 + "|" + "-" * 15]
    lines += [f"{seq_len:>15} | {recall:>14}" for seq_len, recall in rows]
    return "\n".join(lines)


def results_file_name(seq_len: int, run_name: Optional[str]) -> str:
    return f"eval_results_{seq_len}" + (f"_{run_name}" if run_name else "") + ".jsonl"


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model-dir", default="/tmp/model/original")
    ap.add_argument("--seq-len", type=int, default=8192)
    ap.add_argument("--top-k", type=int, default=4096)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--run-name", type=str, default=None)
    ap.add_argument("--local-attn-window", type=int, default=4096)
    ap.add_argument("--data-dir", default="/tmp/data/ruler/niah_multikey_2")
    ap.add_argument("--variant", default="dram", choices=("dram", "quest", "quest_oracle", "full"))
    ap.add_argument("--tokenizer", default="tiktoken", choices=("tiktoken", "bytes"))
    ap.add_argument("--synthetic", type=int, default=0, metavar="N",
                    help="N generated key-value items instead of the data file")
    ap.add_argument("--report", action="store_true", help="print the table over the results files")
    flags = ap.parse_args(argv)
    logging.basicConfig(level=logging.INFO, format="%(asctime)s - %(levelname)s - %(message)s")
    if flags.report:
        print(report("."))
        return 0
    torch.manual_seed(42)
    model = load_model(flags.model_dir, flags.seq_len, variant=flags.variant, top_k=flags.top_k,
                       page_size=flags.page_size, local_attn_window=flags.local_attn_window)
    tokenizer = (ByteTokenizer() if flags.tokenizer == "bytes"
                 else TiktokenTokenizer(str(Path(flags.model_dir) / "tokenizer.model")))
    assert model.params.vocab_size >= tokenizer.n_words
    items = (synthetic_niah(flags.synthetic, max(8, flags.seq_len // 64), 42) if flags.synthetic
             else read_jsonl(f"{flags.data_dir}/validation_{flags.seq_len}.jsonl"))
    recall = evaluate_items(model, tokenizer, items, page_size=flags.page_size,
                            results_path=results_file_name(flags.seq_len, flags.run_name))
    logger.info("Average recall: %s", recall)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
