"""Writes aggregate_loss_cases.json: the literal cases of the reference's loss aggregation test
(tests/rl/common_test.py:457-576), their expected values evaluated from the closed forms that
test states.  Run from the repository root: python tests/golden/make_aggregate_loss_cases.py"""
import json
import os


# The literal cases of tests/rl/common_test.py:457-576 (test_aggregate_loss_values):
# (mode, per-token loss, completion mask, kwargs, expected WeightedMetric.compute()).
_L23, _M23 = [[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]], [[1, 1, 0], [1, 1, 1]]
_L22 = [[0.1, 0.2], [0.3, 0.4]]
AGGREGATE_LOSS_CASES = [
    ("token-mean", _L23, _M23, {}, (0.1 + 0.2 + 0.4 + 0.5 + 0.6) / 5.0),
    ("sequence-mean-token-mean", _L23, _M23, {}, ((0.1 + 0.2) / 2 + (0.4 + 0.5 + 0.6) / 3) / 2),
    ("sequence-mean-token-scale", _L23, _M23, {}, ((0.1 + 0.2) / 3 + (0.4 + 0.5 + 0.6) / 3) / 2),
    ("sequence-mean-token-scale", _L23, _M23, {"norm": 3.14},
     ((0.1 + 0.2) / 3.14 + (0.4 + 0.5 + 0.6) / 3.14) / 2),
    ("sequence-mean-token-sum-norm", _L23, _M23, {}, (0.1 + 0.2 + 0.4 + 0.5 + 0.6) / 2.0),
    ("sequence-mean-token-sum-norm", _L23, _M23, {"norm": 4.0}, (0.1 + 0.2 + 0.4 + 0.5 + 0.6) / 4.0),
    ("token-mean", _L22, [[0, 0], [0, 0]], {}, 0.0),
    ("sequence-mean-token-mean", _L22, [[0, 0], [0, 0]], {}, 0.0),
    ("sequence-mean-token-sum-norm", _L22, [[0, 0], [0, 0]], {"norm": 4.0}, 0.0),
    ("seq-mean-token-sum", _L23, _M23, {}, 0.9),
    ("seq-mean-token-sum", _L22, [[0, 0], [0, 0]], {}, 0.0),
    ("seq-mean-token-sum", _L22, [[1, 1], [0, 0]], {}, 0.3),
    ("sequence-mean-token-sum-norm", _L22, [[1, 1], [0, 0]], {"norm": 4.0}, (0.1 + 0.2) / 4.0),
]

if __name__ == "__main__":
  out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "aggregate_loss_cases.json")
  with open(out, "w") as f:
    json.dump([{"mode": m, "loss": l, "mask": k, "kwargs": kw, "expected": e}
               for m, l, k, kw, e in AGGREGATE_LOSS_CASES], f, indent=1)
