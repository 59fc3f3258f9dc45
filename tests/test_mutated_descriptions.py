"""Well-formed JSON that no graph builder would write: op descriptions mutated in their structure go through the
lowering of the command line tool, which must end with code 0 or with an error code and a message - never by a
signal, and never without an end (an operand read out of bounds, a division by an extent of 0 and products of
extents that wrapped were found this way)."""
import copy
import glob
import json
import os
import random
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
TOOL = os.path.join(ROOT, "akg_amd", "akg-hip")
SOURCES = sorted(glob.glob(os.path.join(ROOT, "akg_amd", "fixtures", "small_*.info")) +
                 glob.glob(os.path.join(HERE, "golden", "ref_info", "*.info")))
EXTENTS = [0, 1, 2, 3, 7, 8, 63, 64, 65, 1000, 4095, 65536, 131073, 2 ** 31 - 1, 2 ** 31, 2 ** 33, 2 ** 40, -1, -2]
TYPES = ["float32", "float16", "bfloat16", "int8", "int32", "int64", "bool", "float64", "uint8", "int16", "complex64", ""]
NAMES = ["Add", "ReduceSum", "ReduceMax", "Transpose", "MatMul", "BatchMatMul", "Reshape", "Cast", "Tile", "Concat", "Gather",
         "UnsortedSegmentSum", "Pad", "StridedSlice", "Slice", "Split", "ArgMax", "Assign", "Select", "BroadcastTo", "Nope"]


def _tensors(node, found):
    if isinstance(node, dict):
        if isinstance(node.get("shape"), list):
            found.append(node)
        for value in node.values():
            _tensors(value, found)
    elif isinstance(node, list):
        for value in node:
            _tensors(value, found)


def mutate(desc, rng):
    """One structural change: an extent replaced everywhere or in one place, a rank changed, an attribute value or an
    element type replaced, an op dropped, doubled or renamed, two tensor names made one, operands or attributes removed."""
    d = copy.deepcopy(desc)
    kind = rng.randrange(9)
    tensors = []
    _tensors(d, tensors)
    ops = d.get("op_desc", [])
    if kind == 0 and tensors:
        values = sorted({v for t in tensors for v in t["shape"] if isinstance(v, int)})
        if values:
            old, new = rng.choice(values), rng.choice(EXTENTS)
            for t in tensors:
                t["shape"] = [new if v == old else v for v in t["shape"]]
    elif kind == 1 and tensors:
        t = rng.choice(tensors)
        if t["shape"]:
            t["shape"][rng.randrange(len(t["shape"]))] = rng.choice(EXTENTS)
    elif kind == 2 and tensors:
        t = rng.choice(tensors)
        if rng.random() < 0.5 and t["shape"]:
            t["shape"].pop(rng.randrange(len(t["shape"])))
        else:
            t["shape"].insert(rng.randrange(len(t["shape"]) + 1), rng.choice(EXTENTS))
    elif kind == 3:
        with_attrs = [o for o in ops if o.get("attr")]
        if with_attrs:
            attr = rng.choice(rng.choice(with_attrs)["attr"])
            value = attr.get("value")
            if isinstance(value, list) and value:
                value[rng.randrange(len(value))] = rng.choice([-5, -1, 0, 1, 2, 3, 7, 100, 2 ** 31, 2 ** 40])
            elif isinstance(value, list):
                attr["value"] = [rng.choice([-1, 0, 5])]
            elif isinstance(value, bool):
                attr["value"] = not value
            elif isinstance(value, (int, float)):
                attr["value"] = rng.choice([-1, 0, 1, 2 ** 31, 1e30, 1e-30])
            else:
                attr["value"] = rng.choice([None, [], "x", 3])
    elif kind == 4 and tensors:
        rng.choice(tensors)["data_type"] = rng.choice(TYPES)
    elif kind == 5 and ops:
        i = rng.randrange(len(ops))
        if rng.random() < 0.5:
            ops.pop(i)
        else:
            ops.insert(i, copy.deepcopy(ops[i]))
    elif kind == 6 and ops:
        rng.choice(ops)["name"] = rng.choice(NAMES)
    elif kind == 7:
        named = [t for t in tensors if "tensor_name" in t]
        if len(named) >= 2:
            a, b = rng.sample(named, 2)
            a["tensor_name"] = b["tensor_name"]
    elif ops:
        op = rng.choice(ops)
        key = rng.choice(["attr", "input_desc", "output_desc"])
        if rng.random() < 0.5:
            op[key] = [] if key != "attr" else None
        elif op.get(key):
            op[key] = op[key][:-1]
    return d


@pytest.mark.parametrize("first", [0, 100, 200])
def test_mutated_descriptions_end_in_a_result_or_an_error_code(first, tmp_path):
    assert os.path.exists(TOOL), "build the command line tool first (make -C akg_amd/csrc)"
    outcomes = {0: 0, 1: 0}
    for seed in range(first, first + 100):
        rng = random.Random(770000 + seed)
        with open(rng.choice(SOURCES), encoding="utf-8") as f:
            desc = json.load(f)
        for _ in range(rng.choice([1, 1, 1, 2, 3])):
            desc = mutate(desc, rng)
        path = str(tmp_path / ("mutant_%d.info" % seed))
        with open(path, "w", encoding="utf-8") as f:
            json.dump(desc, f)
        done = subprocess.run([TOOL, "emit", path], stdout=subprocess.DEVNULL, stderr=subprocess.PIPE, timeout=120)
        assert done.returncode in (0, 1), "seed %d: the tool ended with %d: %s" % (
            seed, done.returncode, done.stderr.decode(errors="replace")[-300:])
        if done.returncode == 1:
            assert b"akg-hip:" in done.stderr, "seed %d: an error code without a message" % seed
        outcomes[done.returncode] += 1
    assert outcomes[0] > 0 and outcomes[1] > 0     # (the mutants are neither all refused nor all harmless)
