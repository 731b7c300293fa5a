"""Consistency of the uncompiled integration/lib/Backends/MI355X sources (they
need a Glow build: LLVM, glog, folly) with the compiled host layer and, where
the reference tree is mounted, with the reference itself:

* every node kind MI355XBackend::shouldLower keeps un-lowered is accepted by
  isOpSupported, and every node kind isOpSupported accepts reaches an
  instruction kind the IR translator (MI355XFunction.cpp) handles;
* every instruction kind the translator emits is a Kind of the host layer
  (glow_amd/host/Program.h), and every host Kind is emitted by it;
* the operand order each host Kind documents is the reference's
  (tools/ClassGen/InstrGen.cpp, CPUSpecificInstrs.h);
* every allow-listed unittest name of make_blacklists.py exists in the
  reference's tests/unittests."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INTEG = os.path.join(ROOT, "integration", "lib", "Backends", "MI355X")
REFERENCE = "/root/reference"

# node kind -> the instruction kind IRGen makes of it, where the names differ
NODE_TO_INST = {
    "Add": "ElementAdd",
    "Save": "Copy", "Reshape": "TensorView",
}
# host kinds that stand for more than one instruction / are produced elsewhere
INST_TO_HOST = {"ElementAdd": "ElementAdd"}


def _read(*parts):
    return open(os.path.join(*parts)).read()


def _function_body(text, signature):
    at = text.index(signature)
    brace = text.index("{", at)
    depth, i = 1, brace + 1
    while depth:
        depth += {"{": 1, "}": -1}.get(text[i], 0)
        i += 1
    return text[brace:i]


def _host_kinds():
    """{name: [operand names]} from the enum in glow_amd/host/Program.h."""
    text = _read(ROOT, "glow_amd", "host", "Program.h")
    body = text[text.index("enum class Kind"):text.index("NumKinds")]
    out = {}
    for name, comment in re.findall(r"^\s*(\w+)(?:\s*=\s*0)?,\s*//\s*(.*)$", body, re.M):
        m = re.match(r"\(([^)]*)\)", comment)
        inner = re.sub(r"\[[^\]]*\]", "", m.group(1)) if m else ""   # drop shapes like [K,N]
        ops = [o.split()[0] for o in inner.split(",") if o.strip()]
        out[name] = ops
    return out


def _backend():
    return _read(INTEG, "MI355XBackend.cpp")


def _supported_nodes():
    body = _function_body(_backend(), "bool MI355XBackend::isOpSupported")
    return set(re.findall(r"Kinded::Kind::(\w+)NodeKind", body))


def _unlowered_nodes():
    body = _function_body(_backend(), "bool MI355XBackend::shouldLower")
    return set(re.findall(r"Kinded::Kind::(\w+)NodeKind", body))


def _translated():
    """{instruction kind: host kind or None} from the translator's switch."""
    text = _read(INTEG, "MI355XFunction.cpp")
    body = _function_body(text, "Error instruction(const Instruction &I)")
    out = {}
    cases = list(re.finditer(r"case Kinded::Kind::(\w+)InstKind:", body))
    for n, c in enumerate(cases):
        end = cases[n + 1].start() if n + 1 < len(cases) else len(body)
        seg = body[c.end():end]
        # add(I, hm::Kind::X, ...) / addInstruction(hm::Kind::X, ...) or one of
        # the host Function's builder shorthands, fn_->createX(...)
        m = re.search(r"hm::Kind::(\w+)|fn_->create(\w+)\(", seg)
        out[c.group(1)] = (m.group(1) or m.group(2)) if m else None
    # consecutive case labels share the code behind the last of them
    names = [c.group(1) for c in cases]
    for i in range(len(names) - 2, -1, -1):
        if out[names[i]] is None and re.fullmatch(
                r"\s*", body[cases[i].end():cases[i + 1].start()]):
            out[names[i]] = out[names[i + 1]]
    return out


def test_unlowered_nodes_are_supported_and_supported_nodes_are_translated():
    supported, unlowered = _supported_nodes(), _unlowered_nodes()
    assert {"Clip", "LeakyRelu", "Relu", "FullyConnected", "Convolution"} <= unlowered
    missing = unlowered - supported
    assert not missing, f"kept from lowering but not accepted by isOpSupported: {missing}"
    translated = _translated()
    for node in sorted(supported):
        inst = NODE_TO_INST.get(node, node)
        assert inst in translated, f"{node}Node is accepted but {inst}Inst is not translated"


def test_translator_and_host_kinds_agree():
    host = _host_kinds()
    translated = _translated()
    memory = {"AllocActivation", "DeallocActivation", "Touch", "TensorView"}
    emitted = set()
    for inst, kind in translated.items():
        if inst in memory:
            continue
        assert kind is not None, f"{inst}Inst is handled without a host kind"
        assert kind in host, f"{inst}Inst -> hm::Kind::{kind}, which Program.h does not have"
        # apart from a few renames an instruction keeps its name
        assert kind == inst, f"{inst}Inst is translated to {kind}"
        emitted.add(kind)
    assert emitted == set(host), f"host kinds no instruction produces: {set(host) - emitted}"
    # the flat C view numbers the kinds in the same order
    py = _read(ROOT, "glow_amd", "host.py")
    count = int(re.search(r"\) = range\((\d+)\)\nACT_NONE", py).group(1))
    assert count == len(host)


def _instr_operands(text):
    """{instruction: [operand names]} of a ClassGen instruction file."""
    out = {}
    for m in re.finditer(r'new(?:BackendSpecific)?Instr\("(\w+)"\)(.*?);', text, re.S):
        out[m.group(1)] = re.findall(r'\.addOperand\("(\w+)"', m.group(2))
    return out


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="reference tree not mounted")
def test_operand_order_is_the_reference_s():
    ref = _instr_operands(_read(REFERENCE, "tools", "ClassGen", "InstrGen.cpp"))
    ref.update(_instr_operands(_read(REFERENCE, "lib", "Backends", "CPU", "ClassGen",
                                     "CPUSpecificInstrs.h")))
    for kind, ops in _host_kinds().items():
        assert kind in ref, f"no {kind}Inst in the reference"
        assert ops == ref[kind], f"{kind}: Program.h says {ops}, the reference {ref[kind]}"


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="reference tree not mounted")
def test_allow_listed_unittests_exist_in_the_reference():
    src = _read(INTEG, "tests", "make_blacklists.py")
    scope = {}
    exec(compile(src[:src.index("HEADER =")], "make_blacklists.py", "exec"), scope)
    for out, allowed in scope["ALLOW"].items():
        source, classes = scope["SUITES"][out]
        text = _read(REFERENCE, "tests", "unittests", source)
        # names written out and names pasted together by the suite's macros
        literal = set(re.findall(r"TEST_P\(\s*\w+\s*,\s*(\w+)\s*\)", text))
        words = set(re.findall(r"\w+", text))
        for name in sorted(allowed):
            if name in literal:
                continue
            # a generated name: every piece between underscores must appear in a
            # macro invocation of the file
            pieces = [p for p in re.split(r"_", name) if p]
            assert all(any(p in w for w in words) for p in pieces), \
                f"{out}: no test {name} in {source}"
        # and the generated black-list does not hide an allowed test
        listed = set(re.findall(r'"(\w+)/0"', _read(INTEG, "tests", out)))
        assert not (allowed & listed), f"{out} black-lists allowed tests: {allowed & listed}"
