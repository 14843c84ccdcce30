"""Writes tests/golden/checkpoint_keys.json: the state-dict schema of a QTIP Llama checkpoint,
derived from the TEXT of the reference's source files (parsed with `ast`, nothing is imported
or executed).  Runs only where /root/reference exists; the JSON it writes is the fixture the
tests read.

  python tests/golden/make_checkpoint_keys.py [/root/reference]

Sources:
  lib/linear/quantized_linear.py  QuantizedLinear.__init__: persistent buffers and parameters
  model/llama.py                  LlamaMLP / LlamaAttention / LlamaDecoderLayer / LlamaModel /
                                  LlamaForCausalLM constructors: sub-module attribute names, which
                                  class each is, and the skip_list token that turns a projection
                                  into a dense nn.Linear
"""
import ast
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def _class(tree, name):
    for node in ast.walk(tree):
        if isinstance(node, ast.ClassDef) and node.name == name:
            return node
    raise KeyError(name)


def _init(cls):
    for node in cls.body:
        if isinstance(node, ast.FunctionDef) and node.name == "__init__":
            return node
    raise KeyError(cls.name + ".__init__")


def _callee(call):
    f = call.func
    if isinstance(f, ast.Attribute):
        return f.attr
    if isinstance(f, ast.Name):
        return f.id
    if isinstance(f, ast.Subscript):  # LLAMA_ATTENTION_CLASSES[...](...)
        return ast.unparse(f.value)
    return ast.unparse(f)


def quantized_linear_state(path):
    """(persistent names in registration order, non-persistent buffer names, conditional names)."""
    tree = ast.parse(open(path).read())
    init = _init(_class(tree, "QuantizedLinear"))
    persistent, transient, conditional = [], [], []

    def visit(stmts, guarded):
        for st in stmts:
            if isinstance(st, ast.If):
                visit(st.body, ast.unparse(st.test))
                visit(st.orelse, "not (" + ast.unparse(st.test) + ")")
                continue
            call = None
            if isinstance(st, ast.Expr) and isinstance(st.value, ast.Call):
                call = st.value
            if call is not None and _callee(call) == "register_buffer":
                name = call.args[0].value
                keep = True
                for kw in call.keywords:
                    if kw.arg == "persistent":
                        keep = bool(kw.value.value)
                (persistent if keep else transient).append(name)
                if guarded and keep:
                    conditional.append([name, guarded])
            if isinstance(st, ast.Assign) and isinstance(st.value, ast.Call) and _callee(st.value) == "Parameter":
                name = st.targets[0].attr
                persistent.append(name)
                if guarded:
                    conditional.append([name, guarded])

    visit(init.body, None)
    return persistent, transient, conditional


def submodules(tree, cls_name):
    """attribute -> {"class": callee, "skip": token or None, "dense_class": callee of the else branch}."""
    init = _init(_class(tree, cls_name))
    out = {}

    def assigns(stmts):
        for st in stmts:
            if isinstance(st, ast.Assign) and isinstance(st.targets[0], ast.Attribute) and \
                    isinstance(st.targets[0].value, ast.Name) and st.targets[0].value.id == "self" and \
                    isinstance(st.value, ast.Call):
                yield st.targets[0].attr, st.value

    for st in init.body:
        if isinstance(st, ast.If):
            m = re.search(r"\{layer_idx\}_(\w+)", ast.unparse(st.test))
            if m and "skip_list" in ast.unparse(st.test):
                for attr, call in assigns(st.body):
                    out[attr] = {"class": _callee(call), "skip": m.group(1)}
                for attr, call in assigns(st.orelse):
                    out[attr]["dense_class"] = _callee(call)
    for attr, call in assigns(init.body):
        callee = _callee(call)
        if callee in ("LlamaMLP", "LlamaRMSNorm", "Embedding", "ModuleList", "Linear", "LlamaModel",
                      "LlamaRotaryEmbedding", "LLAMA_ATTENTION_CLASSES"):
            out[attr] = {"class": callee}
    return out


def main():
    ql_path = os.path.join(REF, "lib/linear/quantized_linear.py")
    persistent, transient, conditional = quantized_linear_state(ql_path)
    tree = ast.parse(open(os.path.join(REF, "model/llama.py")).read())
    schema = {
        "source": ["lib/linear/quantized_linear.py", "model/llama.py"],
        "quantized_linear": {"persistent": persistent, "non_persistent": transient, "conditional": conditional},
        "LlamaMLP": submodules(tree, "LlamaMLP"),
        "LlamaAttention": submodules(tree, "LlamaAttention"),
        "LlamaDecoderLayer": submodules(tree, "LlamaDecoderLayer"),
        "LlamaModel": submodules(tree, "LlamaModel"),
        "LlamaForCausalLM": submodules(tree, "LlamaForCausalLM"),
    }
    # parameter names of the leaf classes (nn.Linear without bias, nn.Embedding, LlamaRMSNorm)
    rms = _init(_class(tree, "LlamaRMSNorm"))
    rms_params = [st.targets[0].attr for st in rms.body
                  if isinstance(st, ast.Assign) and isinstance(st.value, ast.Call) and _callee(st.value) == "Parameter"]
    schema["LlamaRMSNorm"] = {"parameters": rms_params}
    rot = _class(tree, "LlamaRotaryEmbedding")
    rot_buffers = []
    for node in ast.walk(rot):
        if isinstance(node, ast.Call) and _callee(node) == "register_buffer":
            keep = True
            for kw in node.keywords:
                if kw.arg == "persistent":
                    keep = bool(kw.value.value)
            rot_buffers.append([node.args[0].value, keep])
    schema["LlamaRotaryEmbedding"] = {"buffers": rot_buffers}

    # the keys of a 2-layer model with quip_params['skip_list'] = ['1_k', '0_down'] (bias=False, tlut-based code)
    skip = ["1_k", "0_down"]
    ql_keys = [n for n in persistent if n != "bias"]
    keys = []
    top = schema["LlamaForCausalLM"]
    model_attr = [a for a, v in top.items() if v["class"] == "LlamaModel"][0]
    head_attr = [a for a, v in top.items() if v["class"] == "Linear"][0]
    mdl = schema["LlamaModel"]
    for attr, v in mdl.items():
        if v["class"] == "Embedding":
            keys.append(f"{model_attr}.{attr}.weight")
        elif v["class"] == "LlamaRMSNorm":
            keys += [f"{model_attr}.{attr}.{p}" for p in rms_params]
    layers_attr = [a for a, v in mdl.items() if v["class"] == "ModuleList"][0]
    lay = schema["LlamaDecoderLayer"]
    for i in range(2):
        pre = f"{model_attr}.{layers_attr}.{i}."
        for attr, v in lay.items():
            if v["class"] == "LlamaRMSNorm":
                keys += [f"{pre}{attr}.{p}" for p in rms_params]
            else:
                sub = schema["LlamaMLP"] if v["class"] == "LlamaMLP" else schema["LlamaAttention"]
                for pattr, pv in sub.items():
                    if "skip" not in pv:
                        continue
                    if f"{i}_{pv['skip']}" in skip:
                        keys.append(f"{pre}{attr}.{pattr}.weight")
                    else:
                        keys += [f"{pre}{attr}.{pattr}.{n}" for n in ql_keys]
    keys.append(f"{head_attr}.weight")
    schema["example"] = {"num_hidden_layers": 2, "skip_list": skip, "keys": sorted(keys)}
    with open(os.path.join(HERE, "checkpoint_keys.json"), "w") as f:
        json.dump(schema, f, indent=1, sort_keys=True)
    print(f"{len(keys)} keys; QuantizedLinear state: {ql_keys}")


if __name__ == "__main__":
    main()
