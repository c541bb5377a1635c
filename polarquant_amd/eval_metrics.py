"""Scoring functions of the reference's accuracy runs, free of third-party packages.

LongBench's English and code tasks as the reference scores them (utils/metrics.py:12-29, 80-87, 115-131;
test4long.py:142-156) and the GSM8K judge (test4gsm8k.py:33-42).  A score function takes
(prediction, ground_truth, **kwargs) and returns a float in [0, 1]; an example's score is the best
over its reference answers.

`code_sim_score` is `fuzzywuzzy.fuzz.ratio / 100` in the reference.  That package is not required
here: its `ratio` is `round(100 * SequenceMatcher(None, a, b).ratio())`, where the matcher is
difflib's when the optional python-Levenshtein speed-up is absent, and that is what is restated.
With the speed-up installed fuzzywuzzy uses an edit-distance ratio that can differ by a few points
on some string pairs; which of the two the reference's published numbers were made with is not
recorded in its tree.  The Chinese and ROUGE tasks (jieba, rouge) are not among the eight datasets
the reference script runs and are not restated.
"""
from __future__ import annotations

import re
import string
from collections import Counter
from difflib import SequenceMatcher
from typing import Callable, Iterable, List, Optional, Sequence

_PUNCT = frozenset(string.punctuation)
_ARTICLES = re.compile(r"\b(a|an|the)\b")


def normalize_answer(text: str) -> str:
    """Lower case, punctuation dropped, then the articles a / an / the replaced by a blank, blanks collapsed."""
    text = "".join(ch for ch in text.lower() if ch not in _PUNCT)
    return " ".join(_ARTICLES.sub(" ", text).split())


def f1_score(prediction: Sequence, ground_truth: Sequence, **kwargs) -> float:
    """Bag-of-tokens F1: harmonic mean of precision and recall of the multiset overlap."""
    overlap = sum((Counter(prediction) & Counter(ground_truth)).values())
    if overlap == 0:
        return 0.0
    precision, recall = overlap / len(prediction), overlap / len(ground_truth)
    return 2 * precision * recall / (precision + recall)


def qa_f1_score(prediction: str, ground_truth: str, **kwargs) -> float:
    return f1_score(normalize_answer(prediction).split(), normalize_answer(ground_truth).split())


def _ratio(a: str, b: str) -> int:
    """fuzzywuzzy.fuzz.ratio with difflib as the matcher: 100 for equal strings, 0 if one is empty, else the
    rounded percentage."""
    if a == b:
        return 100
    if not a or not b:
        return 0
    return int(round(100 * SequenceMatcher(None, a, b).ratio()))


def code_sim_score(prediction: str, ground_truth: str, **kwargs) -> float:
    """Similarity of the first generated line that is neither a comment nor a code fence to the expected line."""
    first = ""
    for line in prediction.lstrip("\n").split("\n"):
        if "`" not in line and "#" not in line and "//" not in line:
            first = line
            break
    return _ratio(first, ground_truth) / 100


def count_score(prediction: str, ground_truth, **kwargs) -> float:
    """Share of the numbers in the prediction that equal the expected count."""
    numbers = re.findall(r"\d+", prediction)
    return float(sum(n == str(ground_truth) for n in numbers) / len(numbers)) if numbers else 0.0


def retrieval_score(prediction: str, ground_truth: str, **kwargs) -> float:
    """Share of the numbers in the prediction that equal the expected paragraph number ("Paragraph N")."""
    wanted = re.findall(r"Paragraph (\d+)", ground_truth)[0]
    return count_score(prediction, wanted)


def classification_score(prediction: str, ground_truth: str, **kwargs) -> float:
    """1 / (number of class names found in the prediction) if the expected class is among them, else 0; a class
    name that is a proper substring of the expected one does not count as found."""
    found = [c for c in kwargs["all_classes"] if c in prediction]
    # the reference removes from the list it is iterating over, so after a removal the next name is skipped
    i = 0
    while i < len(found):
        if found[i] in ground_truth and found[i] != ground_truth:
            found.remove(found[i])
        i += 1
    return 1.0 / len(found) if ground_truth in found else 0.0


LONGBENCH_METRIC = {
    "narrativeqa": qa_f1_score, "qasper": qa_f1_score, "multifieldqa_en": qa_f1_score,
    "2wikimqa": qa_f1_score, "hotpotqa": qa_f1_score, "musique": qa_f1_score,
    "lcc": code_sim_score, "repobench-p": code_sim_score,
}


def best_score(metric: Callable, prediction: str, answers: Iterable[str], all_classes: Optional[List[str]] = None) -> float:
    """An example's score: the best over its reference answers (test4long.py:150-153)."""
    score = 0.0
    for answer in answers:
        score = max(score, metric(prediction, answer, all_classes=all_classes))
    return score


def extract_single_number(text: str) -> int:
    """The last run of digits in the text, -1 if there is none."""
    runs = re.findall(r"\d+", text)
    return int(runs[-1]) if runs else -1


def judge_gsm8k(output_text: str, answer: str) -> int:
    """1 if the last number on the last line of the generated text is the integer the reference solution ends
    with ("... The answer is 1,234."), else 0."""
    expected = int(answer.split("The answer is ")[1].split(".")[0].strip().replace(",", ""))
    return int(extract_single_number(output_text.split("\n")[-1]) == expected)
