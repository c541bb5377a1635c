"""The LongBench / GSM8K runs (polarquant_amd/accuracy_eval.py) end to end on a toy checkpoint with a byte
tokenizer and synthetic task files: checkpoint -> model -> prompt -> middle truncation -> greedy decode through the
HIP kernels -> score -> result files.  What is checked is the plumbing (the text scored is the text the model
generates for the truncated prompt, the scores are the metric's, the files hold what was returned); the scores
themselves mean nothing on random weights."""
import json

import pytest
import torch

from polarquant_amd import accuracy_eval as ae
from polarquant_amd import checkpoint as ck
from polarquant_amd import eval_metrics as metrics
from polarquant_amd.modeling_common import GenerationConfig, PolarConfig, generate
from polarquant_amd.modeling_llama_polar import LlamaPolarForCausalLM

pytestmark = pytest.mark.gpu


class ByteTokenizer:
    """ids 0..255 are bytes; 256 is the end-of-text token."""

    def encode(self, text):
        return list(text.encode("utf-8"))

    def batch_decode(self, ids, skip_special_tokens=True):
        return [bytes(int(t) for t in row if int(t) < 256).decode("utf-8", errors="replace") for row in ids.tolist()]


@pytest.fixture(scope="module")
def toy(tmp_path_factory, gpu):
    torch.manual_seed(11)
    cfg = PolarConfig(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=2,
                      intermediate_size=256, vocab_size=257, eos_token_id=[256])
    path = str(tmp_path_factory.mktemp("ckpt"))
    ck.save_pretrained(LlamaPolarForCausalLM(cfg), path, shards=2)
    model = ck.load_pretrained(path, torch.bfloat16, gpu)
    return model, ByteTokenizer(), ck.load_generation_config(path)


def _longbench_dir(tmp_path):
    d = tmp_path / "longbench"
    d.mkdir()
    (d / "dataset2prompt.json").write_text(json.dumps({
        "hotpotqa": "Passages:\n{context}\n\nQuestion: {input}\nAnswer:",
        "lcc": "{context}Next line of code:\n"}))
    (d / "dataset2maxlen.json").write_text(json.dumps({"hotpotqa": 6, "lcc": 9}))
    filler = " ".join("word%d" % i for i in range(400))                  # ~2.9 kB: longer than the 700-token limit below
    with open(d / "hotpotqa.jsonl", "w") as f:
        for i in range(3):
            f.write(json.dumps({"context": filler if i else "short passage", "input": "what is %d?" % i,
                                "answers": ["word%d" % i, "w"], "all_classes": None}) + "\n")
    with open(d / "lcc.jsonl", "w") as f:
        for i in range(2):
            f.write(json.dumps({"context": "x = %d\n" % i * 30, "input": "", "answers": ["x = %d" % i], "all_classes": None}) + "\n")
    return d


def test_longbench_run(toy, tmp_path):
    model, tok, gen = toy
    data, out = _longbench_dir(tmp_path), tmp_path / "out"
    log = []
    res = ae.run_longbench(model, tok, gen, str(data), str(out), ["hotpotqa", "lcc"], max_length=700, chat="llama3", progress=log.append)
    again = ae.run_longbench(model, tok, gen, str(data), str(tmp_path / "out2"), ["hotpotqa", "lcc"], max_length=700, chat="llama3")
    assert res == again and set(res) == {"hotpotqa", "lcc"}
    templates = json.loads((data / "dataset2prompt.json").read_text())
    for name, n_new in (("hotpotqa", 6), ("lcc", 9)):
        rows = [json.loads(l) for l in (out / (name + ".jsonl")).read_text().splitlines()]
        examples = [json.loads(l) for l in (data / (name + ".jsonl")).read_text().splitlines()]
        assert [r["idx"] for r in rows] == list(range(len(examples)))
        assert res[name] == pytest.approx(sum(r["score"] for r in rows) / len(rows))
        for r, ex in zip(rows, examples):
            ids = tok.encode(ae.longbench_prompt(templates[name], ex, name, "llama3"))
            if len(ids) > 700:
                ids = ids[:350] + ids[-350:]
            direct = generate(model, torch.tensor([ids], device=model.device), None, gen, max_new_tokens=n_new)
            assert direct.shape[1] <= n_new
            assert r["output_text"] == tok.batch_decode(direct)[0]
            assert r["score"] == metrics.best_score(metrics.LONGBENCH_METRIC[name], r["output_text"], ex["answers"])
            assert 0.0 <= r["score"] <= 1.0 and r["answers"] == ex["answers"]
    # two of the three question prompts were cut to the limit
    assert sum("700 prompt tokens" in line for line in log) == 2


def test_gsm8k_run(toy, tmp_path):
    model, tok, gen = toy
    data = tmp_path / "gsm8k.json"
    with open(data, "w") as f:
        for i in range(3):
            f.write(json.dumps({"conversations": [{"value": "What is %d plus %d?" % (i, i)},
                                                  {"value": "%d+%d=%d\nThe answer is %d" % (i, i, 2 * i, 2 * i)}]}) + "\n")
    out = tmp_path / "res" / "gsm8k.jsonl"
    acc = ae.run_gsm8k(model, tok, gen, str(data), str(out), chat="none", max_new_tokens=12)
    rows = [json.loads(l) for l in out.read_text().splitlines()]
    assert len(rows) == 3 and acc == pytest.approx(sum(r["score"] for r in rows) / 3)
    prefix = ae.gsm8k_prefix(ae.DEFAULT_SHOTS, "none")
    for i, r in enumerate(rows):
        ids = tok.encode(ae.gsm8k_prompt(prefix, "What is %d plus %d?" % (i, i), "none"))
        direct = tok.batch_decode(generate(model, torch.tensor([ids], device=model.device), None, gen, max_new_tokens=12))[0]
        assert r["output_text"] == direct.split("\n\n")[0] and "\n\n" not in r["output_text"]
        assert r["score"] == metrics.judge_gsm8k(r["output_text"], r["answers"])
    assert ae.run_gsm8k(model, tok, gen, str(data), str(out), chat="none", max_new_tokens=12, limit=1) in (0.0, 1.0)
    assert len(out.read_text().splitlines()) == 1


def test_command_line_with_a_tokenizer_directory(tmp_path, gpu, capsys):
    """`python -m polarquant_amd.accuracy_eval ...` as a user runs it: the checkpoint directory also holds the
    tokenizer files (here a byte-level tokenizer without merges, written with the `tokenizers` library)."""
    transformers = pytest.importorskip("transformers")
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    vocab = {ch: i for i, ch in enumerate(sorted(pre_tokenizers.ByteLevel.alphabet()))}
    vocab["<|eot|>"] = 256
    tk = Tokenizer(models.BPE(vocab=vocab, merges=[]))
    tk.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)
    tk.decoder = decoders.ByteLevel()
    ckpt = tmp_path / "ckpt"
    transformers.PreTrainedTokenizerFast(tokenizer_object=tk, eos_token="<|eot|>").save_pretrained(str(ckpt))
    torch.manual_seed(12)
    cfg = PolarConfig(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=1,
                      intermediate_size=128, vocab_size=257, eos_token_id=[256])
    ck.save_pretrained(LlamaPolarForCausalLM(cfg), str(ckpt))
    data = _longbench_dir(tmp_path)
    ae.main(["longbench", "--model", str(ckpt), "--data", str(data), "--out", str(tmp_path / "o"), "--datasets", "lcc",
             "--max-length", "300", "--limit", "1", "--rbits", "3", "--tbits", "3", "--variant", "mixed"])
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert line["task"] == "longbench" and set(line["scores_x100"]) == {"lcc"} and 0 <= line["scores_x100"]["lcc"] <= 100
    assert len((tmp_path / "o" / "lcc.jsonl").read_text().splitlines()) == 1
    gs = tmp_path / "g.json"
    gs.write_text(json.dumps({"conversations": [{"value": "1+1?"}, {"value": "The answer is 2"}]}) + "\n")
    shots = tmp_path / "shots.txt"
    shots.write_text("Question: 2+2?\nLet's think step by step\n2+2=4\nThe answer is 4\n")
    ae.main(["gsm8k", "--model", str(ckpt), "--data", str(gs), "--out", str(tmp_path / "g.jsonl"), "--shots", str(shots),
             "--chat", "none", "--variant", "snapkv"])
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert line["task"] == "gsm8k" and line["accuracy_x100"] in (0.0, 100.0)
