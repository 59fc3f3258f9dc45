"""TEST INFRASTRUCTURE (CPU oracle): attribute reading for the data-movement ops, shared by both restatements.

Rules followed (reference file:line):
  Transpose     perm = value of the second input, else attr "perm"; result dim d = operand dim perm[d]
                (TranslateToMindsporeDialect.cpp:965-979; lowered to tosa.transpose, MindSporeToTosa.cpp:479)
  Tile          multiples = value of the second input, else attr "multiples"; same rank; out[i] = in[i mod extent]
                (TranslateToMindsporeDialect.cpp:1126-1135, MindSporeToLinalg.cpp:970-1040)
  Slice         attrs "begin", "size"; size -1 = up to the end (TranslateToMindsporeDialect.cpp:1089-1101,
                MindSporeFinalizingLower.cpp:125-139)
  StridedSlice  begin / end / strides from attrs or from constant inputs 1..3; a negative end counts from the back;
                extent = ceil((end - begin) / stride); the masks are not used by the lowering
                (TranslateToMindsporeDialect.cpp:1034-1087, MindSporeFinalizingLower.cpp:117-124)
  Pad           attr "padding" = (before, after) pairs, first pair for the LAST dimension, second for the one before,
                ...; attr "value" (integer), constant mode (MindSporeToTosa.cpp:305-376)
  Concat        two operands, attr "axis" (default 0) (TranslateToMindsporeDialect.cpp:1117-1124,
                MindSporeToTosa.cpp:46-58)
  Gather        data, integer indices, axis from a third constant input or attr "axis", batch_dims 0; result shape
                data[:axis] + indices + data[axis+1:], element = data[..., indices[...], ...]
                (TranslateToMindsporeDialect.cpp:1208-1233, MindSporeToLinalg.cpp:526-594). Out-of-range positions are
                undefined in the reference (tensor.extract); both restatements and the kernels clamp them into the axis.
"""

def expand_split(desc):
    """Split -> one Slice per result. The reference translates Split (attr "axis", TranslateToMindsporeDialect.cpp
    :1206-1232) but has no lowering for it, so the meaning restated here is the operator's own: result k is the piece of
    the operand along `axis` that follows the pieces before it, as long as its declared shape says. Returns a
    description without Split entries (the same object if there is none)."""
    if not any(od["name"] == "Split" for od in desc["op_desc"]):
        return desc
    out = dict(desc)
    out["op_desc"] = []
    for od in desc["op_desc"]:
        if od["name"] != "Split":
            out["op_desc"].append(od)
            continue
        attrs = {a["name"]: a["value"] for a in (od.get("attr") or [])}
        src = od["input_desc"][0][0]
        rank = len(src["shape"])
        axis = attrs.get("axis", 0)
        axis = int(axis[0] if isinstance(axis, list) else axis)
        axis = axis + rank if axis < 0 else axis
        offset = 0
        for piece in od["output_desc"]:
            begin = [0] * rank
            begin[axis] = offset
            offset += piece["shape"][axis]
            out["op_desc"].append({
                "name": "Slice", "impl_path": "", "input_desc": [[src]], "output_desc": [piece],
                "attr": [{"data_type": "listInt", "name": "begin", "value": begin},
                         {"data_type": "listInt", "name": "size", "value": list(piece["shape"])}]})
        assert offset == src["shape"][axis], "Split: the results do not cover the operand"
    return out


VIEW_OPS = ("Transpose", "Tile", "Slice", "StridedSlice", "Pad", "Concat", "Gather")


def _ints(v):
    if isinstance(v, (list, tuple)):
        return [int(x) for x in v]
    return [int(v)]


def _from_input_or_attr(od, attrs, idx, key):
    ins = od["input_desc"]
    if len(ins) > idx and "value" in ins[idx][0]:
        return _ints(ins[idx][0]["value"])
    return _ints(attrs[key])


def view_params(od, in_shape):
    """Normalised parameters of op description `od` whose first operand has shape `in_shape`."""
    name = od["name"]
    attrs = {a["name"]: a["value"] for a in (od.get("attr") or [])}
    rank = len(in_shape)
    if name == "Transpose":
        perm = [p + rank if p < 0 else p for p in _from_input_or_attr(od, attrs, 1, "perm")]
        assert sorted(perm) == list(range(rank)), "perm is not a permutation"
        return {"perm": perm}
    if name == "Tile":
        mult = _from_input_or_attr(od, attrs, 1, "multiples")
        assert len(mult) == rank
        return {"multiples": mult}
    if name == "Slice":
        begin, size = _ints(attrs["begin"]), _ints(attrs["size"])
        size = [in_shape[d] - begin[d] if size[d] == -1 else size[d] for d in range(rank)]
        return {"begin": begin, "strides": [1] * rank, "size": size}
    if name == "StridedSlice":
        if "begin" in attrs:
            begin, end, strides = _ints(attrs["begin"]), _ints(attrs["end"]), _ints(attrs["strides"])
        else:
            begin = _from_input_or_attr(od, attrs, 1, "begin")
            end = _from_input_or_attr(od, attrs, 2, "end")
            strides = _from_input_or_attr(od, attrs, 3, "strides")
        end = [e + in_shape[d] if e < 0 else e for d, e in enumerate(end)]
        size = [(end[d] - begin[d] + strides[d] - 1) // strides[d] for d in range(rank)]
        return {"begin": begin, "strides": strides, "size": size}
    if name == "Pad":
        padding = _ints(attrs["padding"])
        low, high = [0] * rank, [0] * rank
        for i in range(len(padding) // 2):
            low[rank - 1 - i], high[rank - 1 - i] = padding[2 * i], padding[2 * i + 1]
        return {"low": low, "high": high, "value": int(attrs.get("value", 0))}
    if name == "Concat":
        axis = attrs.get("axis", 0)
        axis = int(axis[0] if isinstance(axis, list) else axis)
        return {"axis": axis + rank if axis < 0 else axis}
    if name == "Gather":
        ins = od["input_desc"]
        if len(ins) > 2 and "value" in ins[2][0]:
            axis = ins[2][0]["value"]
        else:
            axis = attrs.get("axis", 0)
        axis = int(axis[0] if isinstance(axis, list) else axis)
        assert int(attrs.get("batch_dims", 0)) == 0, "batch_dims other than 0 is not restated"
        return {"axis": axis + rank if axis < 0 else axis}
    raise ValueError("not a data-movement op: %s" % name)
