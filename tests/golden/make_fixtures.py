"""Writes the small golden vectors under tests/golden/ from first principles.

Pure Python (`math` only, double precision): no torch, no oracle, no product
code, so the numbers are independent of everything they are used to check.
The reference's own tests hold no vectors for this path; these are textbook
closed forms evaluated on hand-picked inputs.

    python tests/golden/make_fixtures.py
"""
import json
import math
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def logsumexp(row):
    m = max(row)
    return m + math.log(sum(math.exp(v - m) for v in row))


def ce_case(logits, targets, vocab_start, grad_out):
    """loss_i = logsumexp(x_i) - x_i[t_i] if the target falls into [start, start+V) else
    logsumexp(x_i) - max(x_i); grad = (softmax - onehot*[in range]) * g_i."""
    v = len(logits[0])
    loss, grad = [], []
    for row, t, g in zip(logits, targets, grad_out):
        lse = logsumexp(row)
        tl = t - vocab_start
        ok = 0 <= tl < v
        loss.append(lse - row[tl] if ok else lse - max(row))
        sm = [math.exp(x - lse) for x in row]
        if ok:
            sm[tl] -= 1.0
        grad.append([p * g for p in sm])
    return {"logits": logits, "target": targets, "vocab_start": vocab_start, "grad_output": grad_out,
            "loss": loss, "grad": grad}


def gelu_new(x):
    return 0.5 * x * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def silu(x):
    return x / (1.0 + math.exp(-x))


def main():
    ce = [
        ce_case([[1.0, 2.0, 3.0], [0.5, -1.25, 0.0]], [2, 0], 0, [1.0, 0.5]),
        # -100 and an id past the slice: no one-hot term, loss = lse - max
        ce_case([[0.0, 0.0, 0.0, 0.0], [4.0, -2.0, 1.0, 0.25], [10.0, 9.0, -3.0, 2.0]], [-100, 7, 1], 0,
                [1.0, 1.0, 0.25]),
        # a rank owning vocab [4, 8): target 5 is local index 1, target 2 belongs to another rank
        ce_case([[0.125, 3.0, -0.5, 1.5], [2.0, 2.0, 2.0, 2.0]], [5, 2], 4, [2.0, 1.0]),
        # large magnitudes: the max subtraction must keep this finite
        ce_case([[1000.0, 999.0, 998.0], [-1000.0, -1001.0, -999.5]], [1, 2], 0, [1.0, 1.0]),
    ]
    xs = [-6.0, -3.0, -1.0, -0.5, -1e-3, 0.0, 1e-3, 0.5, 1.0, 2.0, 3.0, 6.0]
    act = {"x": xs, "gelu_new": [gelu_new(x) for x in xs], "silu": [silu(x) for x in xs]}

    # weight sharding (layers.py:78-86) on master[r, c] = 10 r + c, written out by hand:
    # 8 output rows, world 2.  stride 1: rank r keeps rows [4r, 4r+4).  stride 2: chunks of 2 rows,
    # rank r keeps chunks r and r+2 -> rows {2r, 2r+1, 2r+4, 2r+5}.
    shard = {
        "out": 8, "in": 3, "world": 2,
        "column_stride1": {"0": [0, 1, 2, 3], "1": [4, 5, 6, 7]},
        "column_stride2": {"0": [0, 1, 4, 5], "1": [2, 3, 6, 7]},
        # row-parallel over 6 input columns, world 3, stride 1: rank r keeps columns [2r, 2r+2)
        "row_in": 6, "row_world": 3,
        "row_stride1": {"0": [0, 1], "1": [2, 3], "2": [4, 5]},
    }
    for name, obj in (("ce_small.json", ce), ("activations.json", act), ("shard_table.json", shard)):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(obj, f, indent=1)
        print("wrote", name)


if __name__ == "__main__":
    main()
