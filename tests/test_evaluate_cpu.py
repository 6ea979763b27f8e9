"""The recall harness on the CPU: the decoding loop of the evaluation driver
(package and CPU restatement) against a scripted model whose answers are known
by hand, and the bookkeeping around it (answer extraction, results files, the
report table, the byte tokenizer, generated items).  No GPU needed."""

import json
import types

import pytest
import torch

from dram_attention_amd import evaluate as E
from oracle import llama_oracle as M

V = 64
STOP, SPECIAL = 40, 60


class Scripted:
    """Stands in for a model: after a call that ends with token t at position p
    (the position of that last token) the next token is rule(t, p).  Records
    every call as (number of tokens, start_pos)."""

    def __init__(self, rule, max_seq_len=4096, vocab=V):
        self.rule = rule
        self.vocab = vocab
        self.calls = []
        self.params = self.a = types.SimpleNamespace(max_seq_len=max_seq_len)
        self.tok_embeddings = types.SimpleNamespace(weight=torch.zeros(1))

    def forward(self, tokens, start_pos):
        assert tokens.dim() == 2 and tokens.shape[0] == 1
        n = tokens.shape[1]
        self.calls.append((n, start_pos))
        logits = torch.zeros(1, 1, self.vocab)
        logits[0, 0, self.rule(int(tokens[0, -1]), start_pos + n - 1)] = 1.0
        return logits

    __call__ = forward


def both(rule, prefix, suffix, max_gen_len, page_size, max_seq_len=4096):
    a, b = Scripted(rule, max_seq_len), Scripted(rule, max_seq_len)
    got = E.generate(a, prefix, suffix, max_gen_len, page_size=page_size, stop_tokens={STOP},
                     special_start=SPECIAL)
    want = M.greedy_generate(b, prefix, suffix, max_gen_len, page_size, {STOP}, SPECIAL)
    assert a.calls == b.calls
    assert got == want
    return got, a.calls


def test_decoding_loop_by_hand():
    # next = last + 1: the prefix of 37 tokens is prefilled as 32 (two pages of 16); positions
    # 32..41 are fed the prompt (37 + 5 tokens), whatever the model says; from the last
    # prompt token 9 on the model counts up until the length limit
    prefix, suffix = list(range(1, 38)), [5, 6, 7, 8, 9]
    got, calls = both(lambda t, p: t + 1, prefix, suffix, 6, 16)
    assert calls[0] == (32, 0)
    assert calls[1:] == [(1, p) for p in range(32, 47)]      # total_len = 42 + 6 = 48
    # positions 42..47 hold 10..15; the slice ends at the last position fed (46)
    assert got == [10, 11, 12, 13, 14]

    # a stop token ends the run and is not returned: 9 -> 37, 38, 39, 40 (stop)
    got, calls = both(lambda t, p: t + 28 if t == 9 else t + 1, prefix, suffix, 20, 16)
    assert got == [37, 38, 39]
    assert calls[-1] == (1, 44)
    # so does any token of the special range
    got, _ = both(lambda t, p: 61 if t == 11 else t + 1, prefix, suffix, 20, 16)
    assert got == [10, 11]
    # the position reaches the model: next = position
    got, _ = both(lambda t, p: p % 30, prefix, suffix, 4, 16)
    assert got == [41 % 30, 42 % 30, 43 % 30]
    # a stop token inside the prompt ends the run before anything is generated
    got, calls = both(lambda t, p: t + 1, prefix, [5, STOP, 7], 8, 16)
    assert got == [] and calls[-1] == (1, 37)
    # the model's sequence limit caps the run
    got, calls = both(lambda t, p: 3, prefix, suffix, 100, 16, max_seq_len=45)
    assert got == [3, 3] and calls[-1] == (1, 43)
    # page size 8: 37 -> 32 as well; page size 32: one page
    assert both(lambda t, p: t + 1, prefix, suffix, 3, 8)[1][0] == (32, 0)
    assert both(lambda t, p: t + 1, prefix, suffix, 3, 32)[1][0] == (32, 0)
    assert both(lambda t, p: t + 1, list(range(1, 50)), suffix, 3, 16)[1][0] == (48, 0)
    with pytest.raises(AssertionError):
        E.generate(Scripted(lambda t, p: 1), [1, 2, 3], [4], 4, page_size=16, stop_tokens=(),
                   special_start=SPECIAL)


def test_first_number_and_recall_files(tmp_path):
    assert E.first_number(" 4821907.\nThe") == "4821907"
    assert E.first_number("about 12 or 13") == "12"
    assert E.first_number("none") is None
    assert E.results_file_name(8192, None) == "eval_results_8192.jsonl"
    assert E.results_file_name(8192, "quest") == "eval_results_8192_quest.jsonl"
    a = tmp_path / "eval_results_8192.jsonl"
    a.write_text('{"recall": 1}\n{"recall": 0}\nnot json\n{"index": 3}\n{"recall": 1}\n')
    assert E.average_recall(str(a)) == pytest.approx(2 / 3)
    (tmp_path / "eval_results_131072_run.jsonl").write_text('{"recall": 1}\n')
    (tmp_path / "eval_results_16384.jsonl").write_text("")
    assert E.report(str(tmp_path)).split("\n") == [
        "Sequence Length | Average Recall",
        "----------------|---------------",
        "           8192 |         0.6667",
        "          16384 |         0.0000",
        "         131072 |         1.0000",
    ]


def test_byte_tokenizer_and_generated_items():
    tok = E.ByteTokenizer()
    ids = tok.encode("magic número 42\n", bos=True, eos=True)
    assert ids[0] == tok.bos_id and ids[-1] == tok.eos_id and max(ids[1:-1]) < 256
    assert tok.decode(ids) == "magic número 42\n"
    assert tok.special_start == 256 and tok.eos_id in tok.stop_tokens and tok.n_words == 259
    items = E.synthetic_niah(3, 12, seed=5)
    assert items == E.synthetic_niah(3, 12, seed=5) and items != E.synthetic_niah(3, 12, seed=6)
    for i, item in enumerate(items):
        lines = item["input"].split("\n")
        assert item["index"] == i and len(lines) == 13
        assert item["query"] in lines[-1] and lines[-1].endswith("The number is")
        hits = [l for l in lines[:-1] if f" {item['query']} is: " in l]
        assert len(hits) == 1 and hits[0].endswith(f": {item['answer'][0]}.")
        assert len(item["answer"][0]) == 7


def test_evaluate_items_scores_the_first_number(tmp_path):
    """A scripted model that spells " 4217." after the prompt, whatever the prompt: the
    item whose answer is 4217 counts, the other does not; one JSON line per item."""
    tok = E.ByteTokenizer()
    reply = list(b" 4217.") + [tok.eos_id]
    prompt_end = {}

    def rule(t, p):  # position p holds the prompt's last token or a token of the reply
        return reply[min(max(p - prompt_end["at"], 0), len(reply) - 1)]

    items = [{"index": 0, "input": "k one is: 4217.\n" * 3 + "What is one? The number is",
              "query": "one", "answer": ["4217"]},
             {"index": 1, "input": "k two is: 9999.\n" * 3 + "What is two? The number is",
              "query": "two", "answer": ["9999", "1234"]}]
    n = len(tok.encode(items[0]["input"], bos=True, eos=False))
    assert n == len(tok.encode(items[1]["input"], bos=True, eos=False))
    prompt_end["at"] = n - 1
    model = Scripted(rule, vocab=tok.n_words)
    path = tmp_path / "eval_results_64.jsonl"
    recall = E.evaluate_items(model, tok, items, page_size=16, results_path=str(path), max_gen_len=12)
    assert recall == 0.5
    rows = [json.loads(l) for l in path.read_text().splitlines()]
    assert [r["recall"] for r in rows] == [1, 0]
    assert [r["model_output"] for r in rows] == ["4217", "4217"]
    assert rows[1] == {"index": 1, "query": "two", "answer": ["9999", "1234"],
                       "model_output": "4217", "recall": 0}
    assert E.average_recall(str(path)) == 0.5
