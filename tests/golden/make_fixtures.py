#!/usr/bin/env python3
"""Builds the committed golden fixtures from the data files of the reference's own tests.

Reads (never imports or runs) files under /root/reference/tests:
  models/onnx/<Model>.onnx                 binary model files  -> copied to tests/golden/models/
  models/onnx/references/<Model>.ref.hxx   expected outputs    -> numbers extracted into fixtures.json
  alpaka/TestAlpaka*.cxx                   literal input vectors of a few tests -> numbers extracted
  models/generators/generate_input_models.py   its TEST_INPUTS table (the inputs the expected outputs were made from), read
                                           as text: the numbers of each f32([...], shape) entry are extracted
Run in the build container only:  python tests/golden/make_fixtures.py
"""
import json
import os
import re
import shutil

REF = "/root/reference/tests"
HERE = os.path.dirname(os.path.abspath(__file__))

NUM = r"[-+]?(?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?"


def arrays_in(path):
    """{name: [floats]} for every `float name[...] = {...};` and `std::vector<float> name = {...};` in a C++ header."""
    text = open(path).read()
    out = {}
    for m in re.finditer(r"(?:float\s+(\w+)\s*\[[^\]]*\]|std::vector<float>\s+(\w+))\s*=\s*\{(.*?)\}\s*;", text, re.S):
        body = re.sub(r"//[^\n]*", "", m.group(3))
        out[m.group(1) or m.group(2)] = [float(x) for x in re.findall(NUM, re.sub(r"(?<=[\d.])f\b", "", body))]
    return out


def vector_literal(path, test_name, var):
    """The numbers of `std::vector<float> var({ ... })` inside TEST_F(..., test_name)."""
    text = open(path).read()
    start = text.index("TEST_F(SofieAlpakaTest, %s)" % test_name)
    m = re.search(r"std::vector<float>\s+%s\s*\(\s*\{(.*?)\}\s*\)" % var, text[start:], re.S)
    body = re.sub(r"(?<=[\d.])f\b", "", m.group(1))
    return [float(x) for x in re.findall(NUM, body)]


def array_literal(path, test_name, var):
    """The numbers of `std::vector<float> var = { ... }` or `float var[] = { ... }` inside TEST_F(..., test_name)."""
    text = open(path).read()
    start = text.index("TEST_F(SofieAlpakaTest, %s)" % test_name)
    m = re.search(r"(?:std::vector<float>|float)\s+%s\s*(?:\[\])?\s*=\s*\{(.*?)\}" % var, text[start:], re.S)
    body = re.sub(r"(?<=[\d.])f\b", "", m.group(1))
    return [float(x) for x in re.findall(NUM, body)]


def _matching(text, start, open_ch, close_ch):
    """Index just past the bracket that closes the one at text[start]."""
    depth = 0
    for i in range(start, len(text)):
        if text[i] == open_ch:
            depth += 1
        elif text[i] == close_ch:
            depth -= 1
            if depth == 0:
                return i + 1
    raise ValueError("unbalanced brackets")


def test_inputs_table(path, model):
    """The entries of TEST_INPUTS["model"] in the generator script, as [{"kind": "values", "values": [...], "shape": [...]}].
    Only f32(list, shape) entries are understood; anything else (seeded random inputs, integer tensors) returns None."""
    text = open(path).read()
    table = text.index("TEST_INPUTS = {")
    m = re.search(r'\n    "%s": \[' % re.escape(model), text[table:])
    if not m:
        return None
    lst = table + m.end() - 1
    body = text[lst:_matching(text, lst, "[", "]")]
    out, pos = [], 1
    while True:
        c = re.search(r"\b(\w+)\(", body[pos:])
        if not c:
            break
        call_open = pos + c.end() - 1
        call_end = _matching(body, call_open, "(", ")")
        if c.group(1) != "f32":
            return None
        inner = body[call_open + 1:call_end - 1]
        vals_open = inner.index("[") if "[" in inner else 0
        vals_end = _matching(inner, vals_open, "[", "]") if "[" in inner else 0
        values = [float(x) for x in re.findall(NUM, inner[vals_open:vals_end])]
        ar = re.match(r"\s*np\.arange\(\s*(%s)\s*,\s*(%s)\s*\)" % (NUM, NUM), inner)
        if ar:      # f32(np.arange(a, b), shape): the integers from a to b - 1
            values = [float(v) for v in range(int(float(ar.group(1))), int(float(ar.group(2))))]
            vals_end = ar.end()
        shape = [int(x) for x in re.findall(r"\d+", inner[vals_end:])]
        out.append({"kind": "values", "values": values, "shape": shape})
        pos = call_end
    return out


# model -> (expected-array name or None for "the only one", input spec)
IOTA, ONES = {"kind": "iota"}, {"kind": "ones"}
MODELS = {
    "Linear_16": ("all_ones", [ONES]), "Linear_32": ("all_ones", [ONES]), "Linear_64": ("all_ones", [ONES]),
    "LinearWithSigmoid": ("all_ones", [ONES]), "LinearWithSelu": ("all_ones", [ONES]),
    "ConvWithPadding": (None, [IOTA]), "ConvWithoutPadding": (None, [IOTA]), "ConvWithAutopadSameLower": (None, [IOTA]),
    "ConvWithAutopadSameUpper": (None, [IOTA]), "ConvWithStridesPadding": (None, [IOTA]),
    "ConvWithStridesNoPadding": (None, [IOTA]), "ConvWithAsymmetricPadding": (None, [IOTA]),
    "ConvWithDilation": (None, [IOTA]), "ConvWithBias": (None, [IOTA]), "ConvBatch2": (None, [IOTA]),
    "ConvBatch4": (None, [IOTA]), "ConvBatch8": (None, [IOTA]), "ConvGroup2": (None, [IOTA]), "ConvGroup4": (None, [IOTA]),
    "ConvBatch4Group2": (None, [IOTA]), "Conv1d": (None, [IOTA]), "Conv3d": (None, [IOTA]), "GlobalAvgPool2d": (None, [IOTA]),
    "AvgPoolPad": (None, [IOTA]), "AvgPoolCountIncludePad": (None, [IOTA]),
}


def main():
    fixtures = {}
    os.makedirs(os.path.join(HERE, "models"), exist_ok=True)

    def add(model, expected, inputs):
        shutil.copyfile(os.path.join(REF, "models/onnx", model + ".onnx"), os.path.join(HERE, "models", model + ".onnx"))
        os.chmod(os.path.join(HERE, "models", model + ".onnx"), 0o644)
        fixtures[model] = {"inputs": inputs, "expected": expected,
                           "source": "tests/models/onnx/%s.onnx + references/%s.ref.hxx" % (model, model)}

    for model, (arr, inputs) in MODELS.items():
        arrays = arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx"))
        expected = arrays[arr] if arr else next(iter(arrays.values()))
        add(model, expected, inputs)

    # models whose inputs are literal vectors in the reference's test sources
    add("ConvGroupBatch", arrays_in(os.path.join(REF, "models/onnx/references/ConvGroupBatch.ref.hxx"))["output"],
        [{"kind": "values", "values": arrays_in(os.path.join(REF, "models/onnx/references/ConvGroupBatch_input.ref.hxx"))["data"]}])
    un = os.path.join(REF, "alpaka/TestAlpakaElementwiseUnary.cxx")
    for model in ("Gelu", "GeluTanh", "Sqrt", "Reciprocal", "Exp", "Log", "Neg", "Elu", "SeluNonDefaultCoeffs"):
        add(model, next(iter(arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx")).values())),
            [{"kind": "values", "values": vector_literal(un, model, "input")}])
    pool = os.path.join(REF, "alpaka/TestAlpakaPool.cxx")
    for model in ("MaxPool1d", "MaxPool2d", "MaxPool3d", "AvgPool"):
        add(model, arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx"))["output"],
            [{"kind": "values", "values": vector_literal(pool, model, "input")}])
    norm = os.path.join(REF, "alpaka/TestAlpakaNormalization.cxx")
    for model in ("Softmax1d", "Softmax2d", "Softmax3d", "Softmax4d"):
        add(model, arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx"))["output"],
            [{"kind": "values", "values": vector_literal(norm, model, "input_vec")}])
    # models whose inputs are entries of the generator script's TEST_INPUTS table
    gen = os.path.join(REF, "models/generators/generate_input_models.py")
    # (Sub and MaxPool2d_AsymPad are left out: their .ref.hxx files were made from other inputs than the table holds -- 1.5 - 0.25 is
    # not the 1 the file expects -- and the matching outputs exist only in files the reference generates at test time.)
    for model in ("Add", "AddBroadcast2", "AddBroadcast3", "AddBroadcast4", "AddBroadcast5", "AddBroadcast6", "AddBroadcast7", "Mul", "Div", "Pow",
                  "Pow_broadcast", "MaxMultidirectionalBroadcast", "MinMultidirectionalBroadcast", "MeanMultidirectionalBroadcast",
                  "SumMultidirectionalBroadcast", "Tanh", "Erf"):
        inputs = test_inputs_table(gen, model)
        if inputs is None:
            raise RuntimeError("no literal inputs for " + model)
        add(model, next(iter(arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx")).values())), inputs)
    for model in ("LayerNormalization2d", "LayerNormalization4d"):      # expected outputs in <Model>.hxx, not .ref.hxx
        shutil.copyfile(os.path.join(REF, "models/onnx", model + ".onnx"), os.path.join(HERE, "models", model + ".onnx"))
        os.chmod(os.path.join(HERE, "models", model + ".onnx"), 0o644)
        fixtures[model] = {"inputs": test_inputs_table(gen, model), "expected": arrays_in(os.path.join(REF, "models/onnx/references", model + ".hxx"))["output"],
                           "source": "tests/models/onnx/%s.onnx + references/%s.hxx" % (model, model)}
    for model in ("ExpandSameSize", "ExpandDiffSize", "Tile5D", "Gather2d", "GatherAxis0", "GatherAxis1", "GatherAxis2", "GatherAxis3", "GatherNegativeIndices"):
        inputs = test_inputs_table(gen, model)
        if inputs is None:
            raise RuntimeError("no literal inputs for " + model)
        add(model, next(iter(arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx")).values())), inputs)
    # Slice: input and output side by side in the .ref.hxx.  The reference's tests reach them through the namespace inside the file, and two of
    # the files hold each other's namespace (Slice_Neg.ref.hxx declares Slice_Default_Steps and the reverse): the namespace names the model.
    for name in ("Slice", "Slice_Default_Axis", "Slice_Default_Steps", "Slice_Neg"):
        path = os.path.join(REF, "models/onnx/references", name + ".ref.hxx")
        model = re.search(r"namespace\s+(\w+)", open(path).read()).group(1)
        arrays = arrays_in(path)
        add(model, arrays["output"], [{"kind": "values", "values": arrays["input"]}])
        fixtures[model]["source"] = "tests/models/onnx/%s.onnx + references/%s.ref.hxx (namespace %s)" % (model, name, model)
    red = os.path.join(REF, "alpaka/TestAlpakaReduce.cxx")
    for model, var in (("ReduceMean", "input"), ("ReduceProd", "input"), ("ReduceL2", "input"), ("ReduceMax", "input"), ("ReduceMax_axis0", "vals"),
                       ("ReduceMax_mid", "vals")):
        add(model, arrays_in(os.path.join(REF, "models/onnx/references", model + ".ref.hxx"))["output"],
            [{"kind": "values", "values": array_literal(red, model, var)}])
    for model in ("ReduceSum", "ReduceSumSquare"):      # expected outputs are literals of the test itself
        shutil.copyfile(os.path.join(REF, "models/onnx", model + ".onnx"), os.path.join(HERE, "models", model + ".onnx"))
        os.chmod(os.path.join(HERE, "models", model + ".onnx"), 0o644)
        fixtures[model] = {"inputs": [{"kind": "values", "values": array_literal(red, model, "input")}], "expected": array_literal(red, model, "correct"),
                           "source": "tests/models/onnx/%s.onnx + tests/alpaka/TestAlpakaReduce.cxx" % model}
    lin = os.path.join(REF, "alpaka/TestAlpakaLinear.cxx")
    add("LinearWithLeakyRelu", arrays_in(os.path.join(REF, "models/onnx/references/LinearWithLeakyRelu.ref.hxx"))["outputs"],
        [{"kind": "values", "values": vector_literal(lin, "LinearWithLeakyRelu", "input")}])
    bl = os.path.join(REF, "alpaka/TestAlpakaElementwiseBinaryLogic.cxx")
    add("AddBroadcast1", arrays_in(os.path.join(REF, "models/onnx/references/AddBroadcast1.ref.hxx"))["output"],
        [{"kind": "values", "values": vector_literal(bl, "AddBroadcast1", "A_vec")},
         {"kind": "values", "values": vector_literal(bl, "AddBroadcast1", "B_vec")}])

    with open(os.path.join(HERE, "fixtures.json"), "w") as f:
        json.dump(fixtures, f, indent=0, sort_keys=True)
    print("wrote %d fixtures" % len(fixtures))


if __name__ == "__main__":
    main()
