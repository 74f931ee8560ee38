"""Writes tests/golden/hand_traces.json.

Nothing here imports or runs the reference.  Every expected value below was
derived by hand from reading the cited lines of the reference (and, for the
swizzle, copied from the worked example its own files hold); the script only
serialises them so the tests can load them as data.

    python tests/golden/make_fixtures.py
"""
import json
import os

FIXTURES = {
    # tl.swizzle2d docstring example, held by the reference at playground/swizzle.py:12-25:
    # out[new_i][new_j] = i*4+j for size_i = size_j = 4, size_g = 2
    "swizzle_4x4_g2": [[0, 2, 4, 6], [1, 3, 5, 7], [8, 10, 12, 14], [9, 11, 13, 15]],
    # ragged last group, size_i=3, size_j=2, size_g=2: [[i, j, new_i, new_j], ...]
    "swizzle_3x2_g2": [[0, 0, 0, 0], [0, 1, 1, 0], [1, 0, 0, 1], [1, 1, 1, 1], [2, 0, 2, 0], [2, 1, 2, 1]],
    # tritonix/utils/spaces.py:18-19,36-37,50-55
    "spaces": {
        "PowerOfTwo(32,128)": [32, 64, 128], "PowerOfTwo(16,64)": [16, 32, 64], "PowerOfTwo(24,100)": [24, 48, 96],
        "Range(2,5)": [2, 3, 4, 5], "Range(2,8)": [2, 3, 4, 5, 6, 7, 8], "Range(1,10,3)": [1, 4, 7, 10],
        "Choice([4,8])": [4, 8],
    },
    # tritonix/utils/pruners.py:147-169, shape (3, 2)
    "midpoint_3x2": {
        "none": [[1, 1], [1, 0], [0, 1], [0, 0], [2, 1], [2, 0]],
        "after_prune_1_1": [[1, 0], [0, 1], [0, 0], [2, 0]],
        "after_prune_1_1_and_1_0": [[0, 1], [0, 0]],
    },
    "midpoint_order_size4": [2, 1, 3, 0],
    # tritonix/utils/pruners.py:191-225, 1-D space of size 5: [record_idx, value, {idx: pruned?}]
    "unimodal_1d": [
        {"record": [2], "value": 5.0, "pruned": {"0": False, "1": False, "3": False, "4": False}},
        {"record": [3], "value": 7.0, "pruned": {"1": False, "3": True, "4": True}},
        {"record": [1], "value": 4.0, "pruned": {"0": False, "1": False, "2": True, "3": True, "4": True}},
        {"record": [0], "value": 6.0, "pruned": {"0": True, "1": False, "2": True, "3": True, "4": True}},
    ],
    # tritonix/autotune.py:75-140 with a fake launcher; space bm=PowerOfTwo(32,128), ns=Range(2,3), gm=Choice([4,8]),
    # memory_params={"bm"}; the launcher raises OutOfResources iff bm == 128
    "tuner": {
        "timer_A": {"formula": "bm/32 + ns + gm/8",
                    "evaluated": [[64, 2, 4], [64, 2, 8], [64, 3, 4], [64, 3, 8], [32, 2, 4], [32, 2, 8], [32, 3, 4],
                                  [32, 3, 8]],
                    "oom_launches": 0, "best": {"bm": 32, "ns": 2, "gm": 4}},
        "timer_B": {"formula": "4 - bm/64 + ns + gm/8",
                    "evaluated": [[64, 2, 4], [64, 2, 8], [64, 3, 4], [64, 3, 8], [32, 2, 4], [32, 2, 8], [32, 3, 4],
                                  [32, 3, 8]],
                    "oom_launches": 1, "best": {"bm": 64, "ns": 2, "gm": 4}},
        "max_configs_1": {"bm": 64, "ns": 2, "gm": 4},
    },
    # tritonix/dispatcher.py:18-30
    "dispatch_key_c1": [1024, 512, "torch.float16", 512, 768, "torch.float16"],
    # tritonix/ops/matmul.py:169,176,185-193: K=100, block_k=16, split_k=3 -> k ranges loaded by each pid_k
    "splitk_k100_bk16_s3": {"0": [[0, 16], [48, 64], [96, 100]], "1": [[16, 32], [64, 80]], "2": [[32, 48], [80, 96]]},
    # space sizes of the reference's own declarations (Range is inclusive):
    "reference_space_sizes": {"matmul": 432, "splitk": 3024, "glu": 1024},
}

if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hand_traces.json")
    with open(path, "w") as f:
        json.dump(FIXTURES, f, indent=1, sort_keys=True)
    print("wrote", path)
