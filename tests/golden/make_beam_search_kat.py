"""Writes ``beam_search_kat.json``: the known-answer cases of the reference's ``tests/beam_search_test.py`` as data.

Run in the build container (the reference is read as *text*, never imported):

    python tests/golden/make_beam_search_kat.py            # rewrites the fixture
    python tests/golden/make_beam_search_kat.py --check    # compares with the committed fixture, writes nothing

The four transition matrices are parsed out of the reference file with ``ast`` (the ``torch.tensor([...])``
literals at ``:19-66``).  The cases are a transcription of what each reference test sets up and asserts -- the
tests build their arguments in code, so there is nothing to parse them from -- and every number transcribed here
is checked against the numeric literals (and products of literals, ``0.6 * 1e-9``) of the reference lines it
cites: a typo in ``CASES`` fails the run.  ``expected_probs`` are the probabilities whose logarithms the reference
asserts as scores (``np.log(np.array([...]))``), before the division by ``length_norm`` where a length-normalising
scorer is used (``:474-517``).
"""
import argparse
import ast
import json
import os
import re
import sys

REFERENCE = "/root/reference/tests/beam_search_test.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "beam_search_kat.json")

MATRIX_NAMES = {  # reference variable -> key in the fixture
    "transition_probabilities": "T",
    "short_sequence_transition_probabilities": "S",
    "repeated_ngram_transition_probabilities_0": "R0",
    "repeated_ngram_transition_probabilities_1": "R1",
}

COMMENT = "Known-answer cases of the reference's tests/beam_search_test.py, as data: transition matrices (:19-66; rows = last token, START=0, END=5; the step function returns log(matrix[last])), search parameters and the expected sequences of batch element 0 with the probabilities whose logs are the expected scores (divided by length_norm where given). 'reference' cites the lines each case restates."

CASES = [{'name': 'search',
  'reference': 'tests/beam_search_test.py:146-147 (setup :108-116)',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5], [2, 3, 4, 5, 5], [3, 4, 5, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2]},
 {'name': 'batch_size_of_one',
  'reference': 'tests/beam_search_test.py:182-183',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 10,
  'batch_size': 1,
  'expected_top_k': [[1, 2, 3, 4, 5], [2, 3, 4, 5, 5], [3, 4, 5, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2]},
 {'name': 'greedy_search',
  'reference': 'tests/beam_search_test.py:185-193',
  'matrix': 'T',
  'beam_size': 1,
  'max_steps': 50,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5]],
  'expected_probs': [0.4]},
 {'name': 'single_step',
  'reference': 'tests/beam_search_test.py:195-202',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 1,
  'batch_size': 5,
  'expected_top_k': [[1], [2], [3]],
  'expected_probs': [0.4, 0.3, 0.2]},
 {'name': 'early_stopping',
  'reference': 'tests/beam_search_test.py:204-215',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 3,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3], [2, 3, 4], [3, 4, 5]],
  'expected_probs': [0.4, 0.3, 0.2]},
 {'name': 'short_sequence',
  'reference': 'tests/beam_search_test.py:217-231',
  'matrix': 'S',
  'beam_size': 5,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[5, 5, 5, 5, 5], [1, 5, 5, 5, 5], [1, 2, 5, 5, 5], [1, 2, 3, 5, 5], [1, 2, 3, 4, 5]],
  'expected_probs': [0.9, 0.09, 0.009, 0.0009, 0.0001]},
 {'name': 'min_steps_0',
  'reference': 'tests/beam_search_test.py:233-251',
  'matrix': 'S',
  'beam_size': 1,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[5]],
  'expected_probs': [0.9],
  'min_steps': 0},
 {'name': 'min_steps_1',
  'reference': 'tests/beam_search_test.py:253-260',
  'matrix': 'S',
  'beam_size': 1,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 5]],
  'expected_probs': [0.09],
  'min_steps': 1},
 {'name': 'min_steps_2',
  'reference': 'tests/beam_search_test.py:262-269',
  'matrix': 'S',
  'beam_size': 1,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 5]],
  'expected_probs': [0.009],
  'min_steps': 2},
 {'name': 'min_steps_2_beam_3',
  'reference': 'tests/beam_search_test.py:271-278',
  'matrix': 'S',
  'beam_size': 3,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 5, 5, 5], [1, 2, 3, 5, 5], [1, 2, 3, 4, 5]],
  'expected_probs': [0.009, 0.0009, 0.0001],
  'min_steps': 2},
 {'name': 'per_node_beam_size_1',
  'reference': 'tests/beam_search_test.py:280-283',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 50,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5], [2, 3, 4, 5, 5], [3, 4, 5, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2],
  'per_node_beam_size': 1},
 {'name': 'per_node_beam_size_2',
  'reference': 'tests/beam_search_test.py:285-287',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 50,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5], [2, 3, 4, 5, 5], [3, 4, 5, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2],
  'per_node_beam_size': 2},
 {'name': 'length_normalized',
  'reference': 'tests/beam_search_test.py:474-483',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5], [2, 3, 4, 5, 5], [3, 4, 5, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2],
  'length_penalty': 1.0,
  'length_norm': [5, 4, 3]},
 {'name': 'length_penalty_2',
  'reference': 'tests/beam_search_test.py:485-493',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5], [2, 3, 4, 5, 5], [3, 4, 5, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2],
  'length_penalty': 2.0,
  'length_norm': [25, 16, 9]},
 {'name': 'length_penalty_minus_2',
  'reference': 'tests/beam_search_test.py:495-504',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[3, 4, 5, 5, 5], [2, 3, 4, 5, 5], [1, 2, 3, 4, 5]],
  'expected_probs': [0.2, 0.3, 0.4],
  'length_penalty': -2.0,
  'length_norm': [0.1111111111111111, 0.0625, 0.04]},
 {'name': 'length_penalty_2_max_steps_4',
  'reference': 'tests/beam_search_test.py:506-517',
  'matrix': 'T',
  'beam_size': 3,
  'max_steps': 4,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4], [2, 3, 4, 5], [3, 4, 5, 5]],
  'expected_probs': [0.4, 0.3, 0.2],
  'length_penalty': 2.0,
  'length_norm': [16, 16, 9]},
 {'name': 'repeated_ngram_step',
  'reference': 'tests/beam_search_test.py:594-658',
  'matrix': 'R0',
  'beam_size': 2,
  'max_steps': 5,
  'batch_size': 5,
  'expected_top_k': [[1, 3, 1, 3, 1], [1, 2, 3, 1, 3]],
  'expected_probs': [0.36, 0.24]},
 {'name': 'ngram_unigrams',
  'reference': 'tests/beam_search_test.py:660-672',
  'matrix': 'R0',
  'beam_size': 2,
  'max_steps': 3,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3], [1, 3, 5]],
  'expected_probs': [0.4, 6e-10],
  'ngram_size': 1},
 {'name': 'ngram_unigrams_1',
  'reference': 'tests/beam_search_test.py:674-683',
  'matrix': 'R1',
  'beam_size': 2,
  'max_steps': 5,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 4, 5], [1, 2, 4, 3, 5]],
  'expected_probs': [0.00072, 0.00072],
  'ngram_size': 1},
 {'name': 'ngram_bigrams',
  'reference': 'tests/beam_search_test.py:685-698',
  'matrix': 'R0',
  'beam_size': 2,
  'max_steps': 4,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 1], [1, 3, 1, 2]],
  'expected_probs': [0.4, 0.24],
  'ngram_size': 2},
 {'name': 'ngram_trigrams',
  'reference': 'tests/beam_search_test.py:700-713',
  'matrix': 'R0',
  'beam_size': 2,
  'max_steps': 5,
  'batch_size': 5,
  'expected_top_k': [[1, 2, 3, 1, 3], [1, 2, 3, 1, 2]],
  'expected_probs': [0.24, 0.16],
  'ngram_size': 3},
 {'name': 'ngram_end_indices',
  'reference': 'tests/beam_search_test.py:715-731',
  'matrix': 'R0',
  'beam_size': 2,
  'max_steps': 10,
  'batch_size': 5,
  'expected_top_k': [[1, 3, 5, 5], [1, 2, 3, 5]],
  'expected_probs': [6e-10, 4e-10],
  'ngram_size': 1}]


def parse_matrices(source: str) -> dict:
    out = {}
    for node in ast.parse(source).body:
        if isinstance(node, ast.Assign) and len(node.targets) == 1 and isinstance(node.targets[0], ast.Name):
            name = node.targets[0].id
            if name in MATRIX_NAMES and isinstance(node.value, ast.Call) and node.value.args:
                out[MATRIX_NAMES[name]] = ast.literal_eval(node.value.args[0])
    missing = set(MATRIX_NAMES.values()) - set(out)
    if missing:
        raise SystemExit(f"matrices not found in the reference test: {sorted(missing)}")
    return out


def _const(node) -> float:
    """Value of an arithmetic expression of literals (``0.6 * 1e-9``, ``5**2``)."""
    if isinstance(node, ast.Constant) and isinstance(node.value, (int, float)):
        return float(node.value)
    if isinstance(node, ast.UnaryOp) and isinstance(node.op, ast.USub):
        return -_const(node.operand)
    if isinstance(node, ast.BinOp) and isinstance(node.op, (ast.Mult, ast.Div, ast.Pow)):
        a, b = _const(node.left), _const(node.right)
        return a * b if isinstance(node.op, ast.Mult) else (a / b if isinstance(node.op, ast.Div) else a ** b)
    raise ValueError(ast.dump(node))


_NUM = r"-?\d+(?:\.\d+)?(?:e-?\d+)?"


def numbers_in(text: str) -> set:
    """Numeric literals of the text, and the values of the products / quotients / powers of literals written in it."""
    out = {float(t) for t in re.findall(r"(?<![\w.])" + _NUM, text)}
    for m in re.finditer(r"(?<![\w.])" + _NUM + r"(?:\s*(?:\*\*|\*|/)\s*" + _NUM + r")+", text):
        out.add(_const(ast.parse(m.group(0), mode="eval").body))
    return out


def check_case(case: dict, lines: list) -> None:
    """Every transcribed number must occur in the cited lines, in setup_method / _check_results (what a test does not
    pass: ``:108-116``, ``:118-127``), or be one of BeamSearch's own defaults (max_steps 50, beam_size 10:
    ``olmo/beam_search.py:692-693``)."""
    spans = re.findall(r":?(\d+)-(\d+)", case["reference"]) + [("108", "116"), ("118", "127")]
    text = "\n".join("\n".join(lines[int(a) - 1:int(b)]) for a, b in spans)
    have = numbers_in(text) | {0.0, 50.0, 10.0}
    want = set()
    for key in ("expected_top_k", "expected_probs"):
        for row in case[key]:
            want |= {float(v) for v in (row if isinstance(row, list) else [row])}
    for key in ("beam_size", "max_steps", "batch_size", "min_steps", "per_node_beam_size", "ngram_size", "length_penalty"):
        if key in case:
            want.add(float(case[key]))
    stray = {v for v in want if not any(abs(v - h) <= 1e-9 * max(abs(v), abs(h)) for h in have)}
    if stray:
        raise SystemExit(f"case {case['name']}: {sorted(stray)} not among the literals of {case['reference']}")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--check", action="store_true")
    args = ap.parse_args()
    source = open(REFERENCE).read()
    lines = source.splitlines()
    for case in CASES:
        check_case(case, lines)
    fixture = {"_comment": COMMENT, "end_index": 5, "start_token": 0, "rtol": 1e-06, "matrices": parse_matrices(source),
               "cases": CASES}
    if args.check:
        same = json.load(open(OUT)) == fixture
        print("fixture matches" if same else "fixture DIFFERS from what this script writes")
        return 0 if same else 1
    with open(OUT, "w") as f:
        json.dump(fixture, f, indent=1)
        f.write("\n")
    print("wrote", OUT)
    return 0


if __name__ == "__main__":
    sys.exit(main())
