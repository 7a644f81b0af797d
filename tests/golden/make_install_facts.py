"""Writes ``tests/golden/reference_install_facts.json``: what ``spikingjelly_amd.install`` relies on in the reference's
neuron classes, read from the reference's source text with ``ast`` (nothing of the reference is imported or run):

* ``IFNode`` / ``LIFNode`` / ``ParametricLIFNode``: that ``supported_backends`` is a property, the tuples it returns per
  step mode, and the parameter lists of the three forwards that dispatch on the backend string;
* ``MemoryModule``: the parameter lists of ``materialize_states`` and of the ``backend`` setter, and the message of the
  ``NotImplementedError`` the setter raises;
* ``base.check_backend_library``: its parameter list and the messages of the ``ImportError`` s it raises.

Run in the build container (the reference lies at /root/reference there):  python tests/golden/make_install_facts.py
``tests/test_install.py`` checks the stand-in package it installs into, and the methods ``install`` replaces, against
this fixture.
"""

import ast
import json
import os
import sys

REF = os.environ.get("SJ_REFERENCE", "/root/reference/spikingjelly/activation_based")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_install_facts.json")
CLASSES = {"IFNode": "neuron/integrate_and_fire.py", "LIFNode": "neuron/lif.py", "ParametricLIFNode": "neuron/plif.py"}
FORWARDS = ("single_step_functional_forward", "multi_step_functional_forward", "multi_step_forward")


def parameters(fn: ast.FunctionDef) -> list:
    a = fn.args
    names = [x.arg for x in a.posonlyargs + a.args]
    if a.vararg:
        names.append("*" + a.vararg.arg)
    names += [x.arg for x in a.kwonlyargs]
    if a.kwarg:
        names.append("**" + a.kwarg.arg)
    return names


def class_def(tree: ast.Module, name: str) -> ast.ClassDef:
    return next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == name)


def method(cls: ast.ClassDef, name: str, decorator: str = None) -> ast.FunctionDef:
    for n in cls.body:
        if isinstance(n, ast.FunctionDef) and n.name == name:
            decos = [ast.unparse(d) for d in n.decorator_list]
            if decorator is None and not any(d.endswith(".setter") for d in decos):
                return n
            if decorator is not None and decorator in decos:
                return n
    raise KeyError(name)


def backends_by_step_mode(fn: ast.FunctionDef) -> dict:
    """``if self.step_mode == 's': return (...)`` branches of a ``supported_backends`` property."""
    out = {}
    for node in ast.walk(fn):
        if isinstance(node, ast.If) and isinstance(node.test, ast.Compare) and ast.unparse(node.test.left) == "self.step_mode":
            mode = ast.literal_eval(node.test.comparators[0])
            ret = next((s for s in node.body if isinstance(s, ast.Return)), None)
            if ret is not None:
                out[mode] = list(ast.literal_eval(ret.value))
    return out


def raised_messages(fn: ast.FunctionDef, exception: str) -> list:
    msgs = []
    for node in ast.walk(fn):
        if isinstance(node, ast.Raise) and isinstance(node.exc, ast.Call) and ast.unparse(node.exc.func) == exception:
            msgs.append(ast.unparse(node.exc.args[0]))
    return msgs


def main() -> int:
    facts = {"source": "spikingjelly/activation_based (reference), read with ast", "classes": {}}
    for name, rel in CLASSES.items():
        with open(os.path.join(REF, rel)) as f:
            cls = class_def(ast.parse(f.read()), name)
        prop = method(cls, "supported_backends")
        facts["classes"][name] = {
            "file": rel,
            "supported_backends_is_property": "property" in [ast.unparse(d) for d in prop.decorator_list],
            "supported_backends": backends_by_step_mode(prop),
            "forwards": {fw: parameters(method(cls, fw)) for fw in FORWARDS},
        }
    with open(os.path.join(REF, "base.py")) as f:
        tree = ast.parse(f.read())
    mm = class_def(tree, "MemoryModule")
    setter = method(mm, "backend", "backend.setter")
    check = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == "check_backend_library")
    facts["MemoryModule"] = {
        "materialize_states": parameters(method(mm, "materialize_states")),
        "backend_setter": parameters(setter),
        "backend_setter_calls_check_backend_library": any(
            isinstance(n, ast.Call) and ast.unparse(n.func) == "check_backend_library" for n in ast.walk(setter)),
        "backend_setter_not_implemented_message": raised_messages(setter, "NotImplementedError"),
    }
    facts["check_backend_library"] = {"parameters": parameters(check), "import_error_messages": raised_messages(check, "ImportError")}
    with open(OUT, "w") as f:
        json.dump(facts, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"wrote {OUT}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
