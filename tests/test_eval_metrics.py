"""Scoring functions of the accuracy runs (polarquant_amd/eval_metrics.py) against values fixed by their
definitions: hand-counted token overlaps, difflib's published matching-blocks ratio 2M/T, and the literal behaviour
of the reference's lines on the corner cases they have (utils/metrics.py:12-29, 80-87, 88-101, 115-131;
test4gsm8k.py:33-42)."""
import pytest

from polarquant_amd import accuracy_eval as ae
from polarquant_amd import eval_metrics as m


def test_normalize_answer_order_of_steps():
    # punctuation goes before the articles are looked for: "the." is an article, "a-b" becomes one word
    assert m.normalize_answer("The  cat, the.  An a-b!") == "cat ab"
    assert m.normalize_answer("Theatre of an Anthem") == "theatre of anthem"      # articles only as whole words


def test_qa_f1_hand_counted():
    # prediction tokens {paris, is, capital}: 3; truth {paris}: overlap 1 -> p = 1/3, r = 1 -> f1 = 0.5
    assert m.qa_f1_score("Paris is the capital.", "paris") == pytest.approx(0.5)
    # multiset overlap: "no no no" vs "no no" -> overlap 2, p = 2/3, r = 1 -> 0.8
    assert m.qa_f1_score("no no no", "no, no") == pytest.approx(0.8)
    assert m.qa_f1_score("yes", "no") == 0.0
    assert m.qa_f1_score("", "no") == 0.0
    assert m.qa_f1_score("An apple", "the APPLE!") == 1.0


def test_code_sim_first_code_line_and_ratio():
    # the first line without a back-tick, '#' or '//' is compared; leading blank lines are dropped first
    pred = "\n\n```python\n# a comment\n// another\nreturn x + 1\nreturn y\n"
    assert m.code_sim_score(pred, "return x + 1") == 1.0
    # difflib: "abcd" vs "bcde" -> matching block "bcd" (3), ratio 2*3/8 = 0.75
    assert m.code_sim_score("abcd", "bcde") == 0.75
    # rounding to whole per cent: "ab" vs "abc" -> 2*2/5 = 0.8; "a" vs "abc" -> 2/4 = 0.5
    assert m.code_sim_score("ab", "abc") == 0.8
    assert m.code_sim_score("a", "abc") == 0.5
    # every line is a comment -> the empty string is compared: 0, except against an empty expectation (equal strings)
    assert m.code_sim_score("# only\n// comments", "x = 1") == 0.0
    assert m.code_sim_score("# only", "") == 1.0
    # a blank first line after the stripped newlines counts as the first code line
    assert m.code_sim_score("\n \nx = 1", "x = 1") == pytest.approx(m._ratio(" ", "x = 1") / 100)


def test_count_and_retrieval_scores():
    assert m.count_score("there are 3 or maybe 4, no 3", 3) == pytest.approx(2 / 3)
    assert m.count_score("none", 3) == 0.0
    assert m.retrieval_score("Paragraph 12 and 7", "Paragraph 12") == 0.5
    assert m.retrieval_score("120", "Paragraph 12") == 0.0                      # whole numbers, not substrings


def test_classification_score_including_the_skip_after_a_removal():
    classes = ["city", "city name", "country", "river"]
    assert m.classification_score("a country", "country", all_classes=classes) == 1.0
    assert m.classification_score("a country or a river", "country", all_classes=classes) == 0.5
    # "city" is inside "city name": found ["city", "city name"] -> "city" is a proper substring of the truth and is removed
    assert m.classification_score("the city name", "city name", all_classes=classes) == 1.0
    assert m.classification_score("a river", "country", all_classes=classes) == 0.0
    # the reference removes while iterating: with ["ab", "abc", "abcd"] all found and truth "abcd", "ab" is removed,
    # "abc" is skipped by the shift and stays -> 2 names left -> 0.5
    assert m.classification_score("abcd", "abcd", all_classes=["ab", "abc", "abcd"]) == 0.5


def test_best_score_takes_the_best_answer():
    assert m.best_score(m.qa_f1_score, "blue", ["red", "dark blue", "blue"]) == 1.0
    assert m.best_score(m.qa_f1_score, "blue", []) == 0.0


def test_gsm8k_judge():
    assert m.extract_single_number("12 apples and 7 pears") == 7
    assert m.extract_single_number("none") == -1
    sol = "She sells 1,200 + 34.\nThe answer is 1,234."
    assert m.judge_gsm8k("1200+34=1234\nThe answer is 1234", sol) == 1
    assert m.judge_gsm8k("The answer is 1234\nor 1235", sol) == 0             # only the last line is read
    assert m.judge_gsm8k("The answer is 12.5", "The answer is 5") == 1          # the last run of digits: 5
    assert m.judge_gsm8k("no number", "The answer is 5") == 0


def test_truncate_middle():
    ids = list(range(10))
    assert ae.truncate_middle(ids, 10) == ids
    assert ae.truncate_middle(ids, 6) == [0, 1, 2, 7, 8, 9]
    assert ae.truncate_middle(ids, 5) == [0, 1, 8, 9]                           # an odd limit keeps 2 * (5 // 2) tokens


def test_prompts():
    tpl = "Read: {context}\nQ: {input}\nA:"
    ex = {"context": "C", "input": "I", "answers": ["x"]}
    assert ae.longbench_prompt(tpl, ex, "lcc", "llama3") == "Read: C\nQ: I\nA:"               # code tasks: no chat format
    got = ae.longbench_prompt(tpl, ex, "hotpotqa", "llama3")
    assert got.startswith("<|start_header_id|>user<|end_header_id|>\n\nRead: C") and got.endswith("<|start_header_id|>assistant<|end_header_id|>\n\n")
    assert ae.longbench_prompt(tpl, ex, "hotpotqa", "llama2") == "[INST]Read: C\nQ: I\nA:[/INST]"
    shots = "Question: q1?\nLet's think step by step\nr1\nThe answer is 1\n\nQuestion: q2?\nLet's think step by step\nr2\nThe answer is 2"
    prefix = ae.gsm8k_prefix(shots, "none")
    assert prefix == "q1?\nLet's think step by step\nr1\nThe answer is 1\n\nq2?\nLet's think step by step\nr2\nThe answer is 2\n\n"
    assert ae.gsm8k_prompt(prefix, "q3?", "none") == prefix + "q3?\nLet's think step by step\n"
    p3 = ae.gsm8k_prompt(ae.gsm8k_prefix(shots, "llama3"), "q3?", "llama3")
    assert p3.count("<|eot_id|>") == 5 and p3.endswith("<|start_header_id|>assistant<|end_header_id|>\n\nLet's think step by step\n")
    assert len(ae.DEFAULT_SHOTS.split("\n\n")) == 4 and all(b.startswith("Question: ") for b in ae.DEFAULT_SHOTS.split("\n\n"))
    for block in ae.DEFAULT_SHOTS.split("\n\n"):                               # the built-in examples judge themselves right
        assert m.judge_gsm8k(block, block) == 1
