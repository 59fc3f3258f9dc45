"""Descriptions with one open extent (spelled -1) for the tests of kernels that take extents as arguments: made from a
static builder called with a sentinel extent, which is then opened everywhere it occurs."""
import json

from akg_amd import op_desc


def open_extent(text, sentinel):
    """The description `text` with every extent equal to `sentinel` (one number or several) spelled -1 (an open extent)."""
    d = json.loads(text)
    sentinels = tuple(sentinel) if isinstance(sentinel, (tuple, list)) else (sentinel,)

    def walk(x):
        if isinstance(x, dict):
            if "shape" in x:
                x["shape"] = [-1 if n in sentinels else n for n in x["shape"]]
            for v in x.values():
                walk(v)
        elif isinstance(x, list):
            for v in x:
                walk(v)
    walk(d)
    return json.dumps(d)


DYNAMIC_STREAMS = {
    # two float32 column sums of one pass over two bf16 operands (the gradient of a scale and a bias over the tokens)
    "biasgrad_bf16": lambda t, name: op_desc.bias_grad(t, 1024, "bfloat16", name),
    # a column maximum over rows the 16-byte chunks do not divide (the last chunk of a row overlaps its neighbour)
    "colmax_f16": lambda t, name: op_desc.square_reduce([t, 1001], [0], "float16", False, "ReduceMax", name),
    # a whole tensor into one number: sum of squares (float32)
    "sqsum_all_f32": lambda t, name: op_desc.square_reduce([t, 512], [0, 1], "float32", False, "ReduceSum", name),
}


def _norm_absmax_all(t, name):
    # two reductions of a whole tensor with an op behind one of them: its Euclidean norm and its absolute maximum
    b = op_desc.DescBuilder(name)
    x = b.input([t, 384], "float32")
    norm = b.unary("Sqrt", b.reduce("ReduceSum", b.mul(x, x), [0, 1], False))
    return b.dumps([norm, b.reduce("ReduceMax", b.unary("Abs", x), [0, 1], False)])


DYNAMIC_STREAMS["norm_absmax_all_f32"] = _norm_absmax_all


def _declared_half_colsum(t, name):
    b = op_desc.DescBuilder(name)
    return b.dumps([b.reduce("ReduceSum", b.input([t, 192], "float16"), [0], False)])


def _declared_bf16_sum_all(t, name):
    b = op_desc.DescBuilder(name)
    return b.dumps([b.reduce("ReduceSum", b.input([t, 64], "bfloat16"), [0, 1], False)])


# sums declared in a 16-bit type: one serial chain per result in index order, whatever the extent
DYNAMIC_STREAMS["declared_f16_colsum"] = _declared_half_colsum
DYNAMIC_STREAMS["declared_bf16_sum_all"] = _declared_bf16_sum_all


DYNAMIC_COLUMNS = {
    "softmax_classes_f16": lambda n, name: op_desc.softmax_over_axis([n, 21, 32, 48], 1, "float16", name),
    "layernorm_channels_bf16": lambda n, name: op_desc.layernorm_over_axis1(n, 96, 520, "bfloat16", name=name),
}


def _pool_over_tokens(b_, t, name):
    # [batch, tokens, hidden] float16 summed over the tokens in float32, batch and tokens both open
    b = op_desc.DescBuilder(name)
    x = b.cast(b.input([b_, t, 136], "float16"), "float32")
    return b.dumps([b.reduce("ReduceSum", x, [1], False), b.reduce("ReduceMax", x, [1], False)])


def _scaled_pool_over_tokens(b_, t, name):
    # the same with operands that span only some of the extents: a weight per token and a bias per batch entry
    b = op_desc.DescBuilder(name)
    x = b.input([b_, t, 64], "float32")
    w = b.input([1, t, 1], "float32")
    c = b.input([b_, 1, 64], "float32")
    return b.dumps([b.add(b.reduce("ReduceSum", b.mul(x, w), [1], True), c)])


def _rowmax_with_equal_outer_and_inner_extents(b_, t, name):
    # [b, t, b] reduced over its two trailing axes without keep_dims: the result [b] has the extent of the innermost,
    # reduced axis as well as that of the kept one (its size in bytes must follow the kept one)
    b = op_desc.DescBuilder(name)
    x = b.cast(b.input([b_, t, b_], "bfloat16"), "float32")
    return b.dumps([b.cast(b.reduce("ReduceMax", b.mul(x, x), [1, 2], False), "bfloat16")])


# (outer extent, reduced extent) both open: [O, R, I] reduced over R
DYNAMIC_POOLS = {
    "pool_f16": _pool_over_tokens,
    "scaled_pool_f32": _scaled_pool_over_tokens,
    "rowmax_equal_extents_bf16": _rowmax_with_equal_outer_and_inner_extents,
}

# the batch of [N,C,H,W] statistics open: the reduced extent N * H * W is an argument, the channel extent lies between
DYNAMIC_STATS = {
    "bnstats_bf16_16x16": lambda n, name: op_desc.batchnorm_stats(n, 24, 16, 16, "bfloat16", name),
    "bnstats_f32_7x7": lambda n, name: op_desc.batchnorm_stats(n, 40, 7, 7, "float32", name),
}


def _concat_along_the_batch(n, name):
    # an op that works ON the open axis: the two halves of the result come from different operands
    b = op_desc.DescBuilder(name)
    x = b.input([n, 24, 40], "float32")
    y = b.input([n, 24, 40], "float32")
    return b.dumps([b.unary("Neg", op_desc.concat(b, x, y, 0))])


def _tile_along_the_batch(n, name):
    b = op_desc.DescBuilder(name)
    x = b.input([n, 8, 72], "float16")
    return b.dumps([op_desc.tile(b, b.unary("Abs", x), [2, 1, 1])])


# data-movement descriptions with the batch open: (maker, extents opened when the maker is called with 7777, whether the
# source is expected to be the same for every batch size)
DYNAMIC_VIEWS = {
    "transpose_0213_f16": (lambda n, name: op_desc.transpose_0213_neg([n, 128, 12, 64], "float16", name), (7777,), True),
    "transpose_bias_add_bf16": (lambda n, name: op_desc.transpose_bias_add(n, 256, 128, "bfloat16", name), (7777,), True),
    "concat_along_the_batch_f32": (_concat_along_the_batch, (7777, 15554), False),
    "tile_along_the_batch_f16": (_tile_along_the_batch, (7777, 15554), False),
}
