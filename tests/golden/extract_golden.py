#!/usr/bin/env python3
"""Pull the known-answer vectors of the reference's own op tests into JSON fixtures.

Run in the build container (it reads the reference checkout as TEXT; nothing is imported
or executed):

    python tests/golden/extract_golden.py [/root/reference]

For every forward (non-gradient, non-error) `it('<title>', ...)` block of the describe
blocks listed in CASES the script records, in order of appearance, each numeric array
literal of the block (data arrays, shapes, expected values) and each scalar/string
`const` (stride, pad, dilation ...).  The tests under tests/ give each position its
meaning.
Arrays whose elements are not numeric literals are stored as null so positions stay
stable.  Output: tests/golden/<name>.json, one file per reference test file.
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))

# fixture name -> (reference test file, describe blocks to take (None = whole file))
CASES = {
    "matmul": ("tfjs-core/src/ops/matmul_test.ts", ["matmul", "matmulBatch", "dot"]),
    "matmul_webgpu": ("tfjs-webgpu/src/matmul_test.ts", None),
    "fused": ("tfjs-core/src/ops/fused_test.ts", ["fused matmul", "fused conv2d"]),
    "conv2d": ("tfjs-core/src/ops/conv2d_test.ts", ["conv2d"]),
    "depthwise": ("tfjs-core/src/ops/conv2d_depthwise_test.ts", ["depthwiseConv2D"]),
    "separable": ("tfjs-core/src/ops/conv2d_separable_test.ts", ["separableConv2d"]),
    "pool": ("tfjs-core/src/ops/pool_test.ts", ["maxPool", "avgPool", "pool"]),
    "softmax": ("tfjs-core/src/ops/softmax_test.ts", ["softmax"]),
    "reduction": ("tfjs-core/src/ops/reduction_ops_test.ts",
                  ["Reduction: max", "Reduction: min", "Reduction: argmax",
                   "Reduction: argmin", "Reduction: sum", "Reduction: logSumExp"]),
    "unary": ("tfjs-core/src/ops/unary_ops_test.ts",
              ["relu", "clip", "exp", "log", "neg", "abs", "sigmoid", "sqrt", "square",
               "tanh", "rsqrt"]),
    "binary": ("tfjs-core/src/ops/binary_ops_test.ts", ["prelu", "maximum", "minimum"]),
    "arithmetic": ("tfjs-core/src/ops/arithmetic_test.ts", ["add", "sub", "mul", "div"]),
    "gather": ("tfjs-core/src/ops/array_ops_test.ts", ["gather"]),
    "transpose": ("tfjs-core/src/ops/transpose_test.ts", ["transpose"]),
    "dequant": ("tfjs-core/src/io/io_utils_test.ts", ["decodeWeights"]),
    "slice": ("tfjs-core/src/ops/slice_test.ts",
              ["slice1d", "slice2d", "slice3d", "slice4d", "slice5d", "slice6d"]),
    "strided_slice": ("tfjs-core/src/ops/strided_slice_test.ts", ["stridedSlice"]),
    "reverse": ("tfjs-core/src/ops/reverse_test.ts",
                ["reverse1d", "reverse2d", "reverse3d", "reverse4d"]),
    "concat": ("tfjs-core/src/ops/concat_test.ts", ["concat1d", "concat2d", "concat3d"]),
    "pad": ("tfjs-core/src/ops/pad_test.ts", ["pad1d", "pad2d", "pad4d", "pad"]),
    "tile_onehot": ("tfjs-core/src/ops/array_ops_test.ts", ["tile", "oneHot"]),
    "compare": ("tfjs-core/src/ops/compare_ops_test.ts",
                ["equal", "notEqual", "less", "lessEqual", "greater", "greaterEqual"]),
    "logical": ("tfjs-core/src/ops/logical_ops_test.ts",
                ["logicalNot", "logicalAnd", "logicalOr"]),
    "batchnorm": ("tfjs-core/src/ops/batchnorm_test.ts",
                  ["batchNorm4D", "batchNorm3D", "batchNorm2D"]),
    "resize_bilinear": ("tfjs-core/src/ops/resize_bilinear_test.ts", ["resizeBilinear"]),
    "resize_nearest": ("tfjs-core/src/ops/resize_nearest_neighbor_test.ts",
                       ["resizeNearestNeighbor"]),
    "where": ("tfjs-core/src/ops/logical_ops_test.ts", ["where"]),
    "where_async": ("tfjs-core/src/ops/logical_ops_test.ts", ["whereAsync"]),
    "array_extra": ("tfjs-core/src/ops/array_ops_test.ts",
                    ["stack", "unstack", "split", "expandDims"]),
    "mean": ("tfjs-core/src/ops/reduction_ops_test.ts", ["Reduction: mean"]),
    "unary_extra": ("tfjs-core/src/ops/unary_ops_test.ts",
                    ["step", "logSigmoid", "softplus", "reciprocal", "log1p", "ceil", "floor", "sign",
                     "isNaN", "isInf", "isFinite", "expm1", "sin", "cos", "tan", "asin", "acos",
                     "atan", "sinh", "cosh", "leakyRelu", "elu", "selu", "round", "asinh", "acosh",
                     "atanh", "erf"]),
    "binary_extra": ("tfjs-core/src/ops/binary_ops_test.ts",
                     ["squaredDifference", "mod", "atan2"]),
    "arithmetic_extra": ("tfjs-core/src/ops/arithmetic_test.ts", ["pow", "addN"]),
    "lrn": ("tfjs-core/src/ops/lrn_test.ts", ["localResponseNormalization with Tensor3D",
                                              "localResponseNormalization with Tensor4D"]),
    "cumsum": ("tfjs-core/src/ops/array_ops_test.ts", ["cumsum"]),
    "topk": ("tfjs-core/src/ops/topk_test.ts", ["topk"]),
    "space_batch_depth": ("tfjs-core/src/ops/array_ops_test.ts",
                          ["batchToSpaceND", "spaceToBatchND", "depthToSpace"]),
    "optimizer_sgd": ("tfjs-core/src/optimizers/sgd_optimizer_test.ts", None),
    "optimizer_momentum": ("tfjs-core/src/optimizers/momentum_optimizer_test.ts", None),
    "optimizer_adagrad": ("tfjs-core/src/optimizers/adagrad_optimizer_test.ts", None),
    "optimizer_adadelta": ("tfjs-core/src/optimizers/adadelta_optimizer_test.ts", None),
    "optimizer_adam": ("tfjs-core/src/optimizers/adam_optimizer_test.ts", None),
    "optimizer_adamax": ("tfjs-core/src/optimizers/adamax_optimizer_test.ts", None),
    "optimizer_rmsprop": ("tfjs-core/src/optimizers/rmsprop_optimizer_test.ts", None),
    "reduction_extra": ("tfjs-core/src/ops/reduction_ops_test.ts",
                        ["Reduction: prod", "Reduction: all", "Reduction: any",
                         "Reduction: moments", "Reduction: norm"]),
    "gather_nd": ("tfjs-core/src/ops/gather_nd_test.ts", ["gatherND"]),
    "scatter_nd": ("tfjs-core/src/ops/scatter_nd_test.ts", ["scatterND"]),
    "sparse_to_dense": ("tfjs-core/src/ops/sparse_to_dense_test.ts", ["sparseToDense"]),
    "segment": ("tfjs-core/src/ops/segment_ops_test.ts", ["unsortedSegmentSum"]),
    "image": ("tfjs-core/src/ops/image_ops_test.ts", ["nonMaxSuppression", "cropAndResize"]),
    "diag": ("tfjs-core/src/ops/diag_test.ts", ["diag"]),
    "conv3d": ("tfjs-core/src/ops/conv3d_test.ts", ["conv3d"]),
    "pool3d": ("tfjs-core/src/ops/pool_test.ts", ["maxPool3d", "avgPool3d"]),
    "linspace_range": ("tfjs-core/src/ops/array_ops_test.ts", ["linspace", "range"]),
}
# fixture name -> (reference test file, describe blocks, title filter): the gradient blocks,
# whose expected values pin the backward kernels (conv2dDerInput / conv2dDerFilter behind
# tf.grads of conv2d and behind conv2dTranspose, the depthwise and pooling backprops).  A
# describe's beforeEach block is recorded as a case titled "beforeEach".
GRAD_CASES = {
    "conv2d_grad": ("tfjs-core/src/ops/conv2d_test.ts", ["conv2d"], r"^gradient"),
    "conv2d_transpose": ("tfjs-core/src/ops/conv2d_transpose_test.ts", ["conv2dTranspose"],
                         r"^(input=|gradient)"),
    "depthwise_grad": ("tfjs-core/src/ops/conv2d_depthwise_test.ts",
                       ["depthwiseConv2d gradients"], r"^(beforeEach|wrt )"),
    "pool_grad": ("tfjs-core/src/ops/pool_test.ts", ["maxPoolBackprop", "avgPool", "poolBackprop"],
                  r"gradient"),
    "resize_bilinear_grad": ("tfjs-core/src/ops/resize_bilinear_test.ts", ["resizeBilinear gradients"],
                             r"^(greyscale|color)"),
    "resize_nearest_grad": ("tfjs-core/src/ops/resize_nearest_neighbor_test.ts",
                            ["resizeNearestNeighbor gradients"], r"^(greyscale|color)"),
}
# blocks whose title matches are not forward known-answer cases
SKIP = re.compile(r"grad|throw|raises|tensor-like|TensorLike|does not match|do not match|"
                  r"dont match|non-tensor|string tensor|Unsupported|error", re.I)

_NUM = re.compile(r"[-+]?(?:NaN|Infinity|(?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?)")


_CONST = re.compile(r"\bconst\s+([A-Za-z_$][\w$]*)(?::[^=;]+)?\s*=\s*"
                    r"(?:(-?\d+\.?\d*(?:[eE][-+]?\d+)?)|'([^']*)'|(true|false))\s*;")


def _match_paren(src, j):
    """src[j-1] == '(' ; return index just past the matching ')'."""
    depth, in_str = 1, None
    while j < len(src) and depth:
        c = src[j]
        if in_str:
            if c == "\\":
                j += 1
            elif c == in_str:
                in_str = None
        elif c in "'\"`":
            in_str = c
        elif c == "/" and src[j + 1] == "/":
            j = src.index("\n", j)
        elif c == "(":
            depth += 1
        elif c == ")":
            depth -= 1
        j += 1
    return j


def blocks_of(src, describes, before_each=False):
    """Yield (describe, title, body) for each it() block of the wanted describe blocks (and,
    on request, for their beforeEach blocks under the title "beforeEach")."""
    scopes = []
    for m in re.finditer(r"\bdescribe\w*\(\s*['\"]([^'\"]*)['\"]", src):
        end = _match_paren(src, src.index("(", m.start()) + 1)
        scopes.append((m.group(1), m.start(), end))
    if not scopes:
        scopes = [(None, 0, len(src))]
    for name, start, end in scopes:
        if describes is not None and name not in describes:
            continue
        for m in re.finditer(r"\bit\(\s*(['\"])((?:(?!\1)[^\\]|\\.)*)\1\s*,", src[start:end]):
            j = start + m.start()
            stop = _match_paren(src, src.index("(", j) + 1)
            yield name, m.group(2), src[start + m.end():stop]
        for m in re.finditer(r"\bbeforeEach\(", src[start:end] if before_each else ""):
            j = start + m.start()
            stop = _match_paren(src, src.index("(", j) + 1)
            yield name, "beforeEach", src[j:stop]


def consts_of(body):
    out = {}
    for m in _CONST.finditer(body):
        if m.group(2) is not None:
            t = m.group(2)
            out[m.group(1)] = float(t) if re.search(r"[.eE]", t) else int(t)
        elif m.group(3) is not None:
            out[m.group(1)] = m.group(3)
        else:
            out[m.group(1)] = m.group(4) == "true"
    return out


def parse_array(body, i):
    """Parse a bracketed literal starting at body[i]=='['. Returns (value|None, end)."""
    assert body[i] == "["
    out, ok = [], True
    i += 1
    while True:
        while i < len(body) and body[i] in " \t\r\n,":
            i += 1
        if body.startswith("//", i):
            i = body.index("\n", i)
            continue
        if body[i] == "]":
            return (out if ok else None), i + 1
        if body[i] == "[":
            v, i = parse_array(body, i)
            if v is None:
                ok = False
            out.append(v)
            continue
        m = _NUM.match(body, i)
        nxt = body[m.end()] if m and m.end() < len(body) else ""
        if m and (nxt in " \t\r\n,]"):
            t = m.group(0)
            out.append(float(t) if re.search(r"[.eEN]|Infinity", t) else int(t))
            i = m.end()
            continue
        m2 = re.match(r"(true|false)\b", body[i:])
        if m2:
            out.append(1 if m2.group(1) == "true" else 0)
            i += m2.end()
            continue
        # not a literal element: skip to the matching close, mark the array unusable
        ok = False
        depth = 0
        while True:
            c = body[i]
            if c in "([{":
                depth += 1
            elif c in ")]}":
                if depth == 0:
                    break
                depth -= 1
            elif c == "," and depth == 0:
                break
            i += 1


def arrays_of(body):
    res, i = [], 0
    while i < len(body):
        c = body[i]
        if c in "'\"`":  # skip strings
            j = i + 1
            while body[j] != c:
                j += 2 if body[j] == "\\" else 1
            i = j + 1
            continue
        if body.startswith("//", i):
            i = body.index("\n", i)
            continue
        if c == "[":
            k = i - 1
            while k >= 0 and body[k] in " \t\r\n":
                k -= 1
            prev = body[k] if k >= 0 else ""
            if prev.isalnum() or prev in "_)]>":  # indexing / type syntax, not a literal
                v, j = parse_array(body, i)
                i = j
                continue
            v, j = parse_array(body, i)
            res.append(v)
            i = j
            continue
        i += 1
    return res


def _eval_expr(tok, env):
    """Evaluate a literal / identifier / array-of-those from the conv_util tests."""
    tok = tok.strip()
    if tok.startswith("["):
        inner, parts, depth, cur = tok[1:-1], [], 0, ""
        for ch in inner:
            if ch == "[":
                depth += 1
            elif ch == "]":
                depth -= 1
            if ch == "," and depth == 0:
                parts.append(cur)
                cur = ""
            else:
                cur += ch
        if cur.strip():
            parts.append(cur)
        return [_eval_expr(p, env) for p in parts]
    if tok in ("null", "undefined"):
        return None
    if tok in ("true", "false"):
        return tok == "true"
    if tok[0] in "'\"":
        return tok[1:-1]
    if re.fullmatch(r"-?\d+", tok):
        return int(tok)
    if re.fullmatch(r"-?\d*\.\d+", tok):
        return float(tok)
    if tok in env:
        return env[tok]
    raise KeyError(tok)


def _split_args(s):
    parts, depth, cur = [], 0, ""
    for ch in s:
        if ch in "[(":
            depth += 1
        elif ch in "])":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        parts.append(cur)
    return parts


_DECL = re.compile(r"\bconst\s+([A-Za-z_$][\w$]*)\s*(?::[^=]+?)?=\s*([^;]+);")


def extract_conv_util():
    """ops/conv_util_test.ts: every computeConv2DInfo / computePool2DInfo call with literal
    arguments, and the fields the test expects of the result (or that it must throw)."""
    rel = "tfjs-core/src/ops/conv_util_test.ts"
    src = open(os.path.join(REF, rel)).read()
    out = {"source": rel, "cases": []}
    for m in re.finditer(r"\bdescribe\(\s*'([^']*)'", src):
        name = m.group(1)
        if "3D" in name or "3d" in name or "convertConv2DDataFormat" in name:
            continue
        end = _match_paren(src, src.index("(", m.start()) + 1)
        body = src[m.start():end]
        first_it = body.find("it(")
        env0 = {}
        for d in _DECL.finditer(body[:first_it]):
            try:
                env0[d.group(1)] = _eval_expr(" ".join(d.group(2).split()), env0)
            except KeyError:
                pass
        for it in re.finditer(r"\bit\(\s*'([^']*)'\s*,", body):
            stop = _match_paren(body, body.index("(", it.start()) + 1)
            blk = body[it.end():stop]
            env = dict(env0)
            for d in _DECL.finditer(blk):
                try:
                    env[d.group(1)] = _eval_expr(" ".join(d.group(2).split()), env)
                except (KeyError, IndexError):
                    pass
            call = re.search(r"conv_util\.(computeConv2DInfo|computePool2DInfo)\(", blk)
            if not call:
                continue
            cend = _match_paren(blk, call.end())
            try:
                args = [_eval_expr(" ".join(a.split()), env)
                        for a in _split_args(blk[call.end():cend - 1])]
            except KeyError:
                continue
            expect = {}
            for e in re.finditer(r"expect\(\w+\.([\w.]+)\)\s*\.(?:toEqual|toBe)\(([^;]+)\);", blk):
                try:
                    expect[e.group(1)] = _eval_expr(" ".join(e.group(2).split()), env)
                except KeyError:
                    pass
            out["cases"].append({"describe": name, "title": it.group(1), "fn": call.group(1),
                                 "args": args, "throws": "toThrowError" in blk,
                                 "expect": expect})
    path = os.path.join(OUT, "conv_util.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
        f.write("\n")
    print("conv_util", len(out["cases"]), "cases", os.path.getsize(path), "bytes")


def main():
    extract_conv_util()
    for name, (rel, describes) in CASES.items():
        src = open(os.path.join(REF, rel)).read()
        out = {"source": rel, "cases": []}
        for describe, title, body in blocks_of(src, describes):
            if SKIP.search(title):
                continue
            out["cases"].append({"describe": describe, "title": title,
                                 "consts": consts_of(body), "arrays": arrays_of(body)})
        path = os.path.join(OUT, name + ".json")
        with open(path, "w") as f:
            json.dump(out, f, separators=(",", ":"))
            f.write("\n")
        print(name, len(out["cases"]), "cases", os.path.getsize(path), "bytes")
    for name, (rel, describes, keep) in GRAD_CASES.items():
        src = open(os.path.join(REF, rel)).read()
        out = {"source": rel, "cases": []}
        for describe, title, body in blocks_of(src, describes, before_each=True):
            if not re.search(keep, title) or re.search(r"throw|tensor-like", title, re.I):
                continue
            out["cases"].append({"describe": describe, "title": title,
                                 "consts": consts_of(body), "arrays": arrays_of(body)})
        path = os.path.join(OUT, name + ".json")
        with open(path, "w") as f:
            json.dump(out, f, separators=(",", ":"))
            f.write("\n")
        print(name, len(out["cases"]), "cases", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
