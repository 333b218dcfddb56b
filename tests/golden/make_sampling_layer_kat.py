"""Writes tests/golden/sampling_layer_kat.json: the known-answer tables of the reference's layer test
(tests/unittests/test_sampling_layer.cu:72-92, :151-156, :318-592) transcribed as data. Nothing is
imported or executed from the reference; the tables below were read off its source.
Each expected entry is the set of token ids any uniform draw may produce for (step, batch row).
"""
import json
import os

NEG = "-FLT_MAX"
LOGITS = [
    [-0.9163, -1.2040, -1.6094, -2.3026, NEG, NEG, NEG, NEG],
    [NEG, NEG, NEG, NEG, -0.9163, -1.2040, -1.6094, -2.3026],
    [NEG, NEG, -0.9163, -1.2040, -1.6094, -2.3026, NEG, NEG],
]


def rep(sets):
    """the same per-row pattern at steps 0, 1, 2 with the arg-max at ids 0, 4, 2"""
    return [[[i + off for i in s] for s in sets] for off in (0, 4, 2)]


CASES = []


def case(name, top_k=None, top_p=None, expected=None, local_batch=False):
    CASES.append(dict(name=name, top_k=top_k, top_p=top_p, expected=expected, use_local_batch=local_batch))


case("TopK", top_k=[2], expected=rep([[0, 1]] * 6))
case("BatchTopK", top_k=[2, 1, 1, 2, 1, 1], expected=rep([[0, 1], [0], [0], [0, 1], [0], [0]]))
case("TopP", top_p=[0.3], expected=rep([[0]] * 6))
case("BatchTopP", top_p=[0.3, 0.5, 0.5, 0.3, 0.5, 0.5], expected=rep([[0], [0, 1], [0, 1], [0], [0, 1], [0, 1]]))
case("TopKTopP", top_k=[2], top_p=[0.3], expected=rep([[0]] * 6))
case("BatchTopKTopP", top_k=[2, 2, 1, 2, 2, 1], top_p=[0.3], expected=rep([[0]] * 6))
case("TopKBatchTopP", top_k=[2], top_p=[0.5, 0.3, 0.5, 0.5, 0.3, 0.5],
     expected=rep([[0, 1], [0], [0, 1], [0, 1], [0], [0, 1]]))
case("BatchTopKBatchTopP", top_k=[2, 2, 0, 2, 2, 0], top_p=[0.0, 0.3, 0.5, 0.0, 0.3, 0.5],
     expected=rep([[0, 1], [0], [0, 1], [0, 1], [0], [0, 1]]))
case("InvalidArgsZeroTopK", top_k=[0], expected=rep([[0]] * 6))
case("InvalidArgsZeroTopP", top_p=[0.0], expected=rep([[0]] * 6))
case("InvalidArgsZeroTopKTopP", top_k=[0], top_p=[0.0], expected=rep([[0]] * 6))
case("InvalidArgsZeroBatchTopKTopP", top_k=[0] * 6, top_p=[0.0], expected=rep([[0]] * 6))
case("InvalidArgsZeroTopKBatchTopP", top_k=[0], top_p=[0.0] * 6, expected=rep([[0]] * 6))
case("InvalidArgsBatchTopKContainZero", top_k=[2, 1, 0, 0, 2, 1], expected=rep([[0, 1], [0], [0], [0], [0, 1], [0]]))
case("InvalidArgsBatchTopPContainZero", top_p=[0.5, 0.5, 0.0, 0.5, 0.0, 0.3],
     expected=rep([[0, 1], [0, 1], [0], [0, 1], [0], [0]]))
case("InvalidArgsBatchTopKTopPContainZero", top_k=[2, 2, 1, 0, 2, 0], top_p=[0.0],
     expected=rep([[0, 1], [0, 1], [0], [0], [0, 1], [0]]))
case("InvalidArgsTopKBatchTopPContainZero", top_k=[0], top_p=[0.0, 0.3, 0.5, 0.0, 0.3, 0.5],
     expected=rep([[0], [0], [0, 1], [0], [0], [0, 1]]))
case("InvalidArgsBatchTopKBatchTopPContainZero", top_k=[0, 2, 1, 2, 2, 0], top_p=[0.0, 0.3, 0.9, 0.0, 0.3, 0.5],
     expected=rep([[0], [0], [0], [0, 1], [0], [0, 1]]))
# local-batch cases run ite = 1 with local_batch_size = batch / 3 = 2: only rows 2 and 3 are sampled,
# every other entry of output_ids keeps its initial 0
case("LocalBatchBatchTopP", top_p=[0.3, 0.5, 0.5, 0.3, 0.5, 0.5], local_batch=True,
     expected=[[[0], [0], [0, 1], [0], [0], [0]], [[0], [0], [4, 5], [4], [0], [0]],
               [[0], [0], [2, 3], [2], [0], [0]]])
case("LocalBatchBatchTopKBatchTopP", top_k=[2, 2, 0, 2, 2, 0], top_p=[0.0, 0.3, 0.5, 0.0, 0.3, 0.5], local_batch=True,
     expected=[[[0], [0], [0, 1], [0, 1], [0], [0]], [[0], [0], [4, 5], [4, 5], [0], [0]],
               [[0], [0], [2, 3], [2, 3], [0], [0]]])

if __name__ == "__main__":
    doc = dict(source="tests/unittests/test_sampling_layer.cu:72-92 (shape constants), :151-156 (logits), "
                      ":318-592 (expected id sets)",
               batch_size=6, vocab_size=8, end_id=7, max_input_len=0, max_output_len=3, max_seed=30,
               logits_per_step=LOGITS, cases=CASES)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sampling_layer_kat.json")
    with open(out, "w") as f:
        json.dump(doc, f, indent=1)
    print("wrote", out, len(CASES), "cases")
