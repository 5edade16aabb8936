"""Resolves the shipped vendor package through the reference's OWN operator registry and records the result.

Run in the build container only (it needs /root/reference):

    python tests/golden/make_registry_golden.py

Loads exactly one reference file by path, src/flag_attn/runtime/backend/op_registry.py (plain Python, no
kernels, no device), makes flagattention_amd/upstream_vendor/_amd importable under the module name the
registry asks for ("flag_attn.runtime.backend._amd"), and calls resolve_operator(name, ..., vendor="amd") for
the three operator names of the SageAttention path plus one the package does not declare.  Writes
tests/golden/registry_golden.json: operator name -> [module, qualified name] of what the registry returned.
"""
import importlib.util
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REGISTRY = "/root/reference/src/flag_attn/runtime/backend/op_registry.py"
BACKEND_NAME = "flag_attn.runtime.backend._amd"
OPERATORS = {  # operator name -> generic symbol the reference's facade passes (sage_attention/__init__.py:17-21)
    "sage_attention": "forward",
    "sage_attention_forward": "forward",
    "sage_attention_per_block_int8": "per_block_int8",
}


def resolve_with_reference_registry():
    if ROOT not in sys.path:
        sys.path.insert(0, ROOT)
    spec = importlib.util.spec_from_file_location("reference_op_registry_under_test", REGISTRY)
    registry = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(registry)
    shipped = os.path.join(ROOT, "flagattention_amd", "upstream_vendor", "_amd", "__init__.py")
    bspec = importlib.util.spec_from_file_location(BACKEND_NAME, shipped)
    backend = importlib.util.module_from_spec(bspec)
    saved = sys.modules.get(BACKEND_NAME)
    sys.modules[BACKEND_NAME] = backend  # import_module returns an already loaded module without touching its parents
    try:
        bspec.loader.exec_module(backend)
        out = {}
        for name, generic in OPERATORS.items():
            # the generic module named here does not exist: the override must win before it is looked at
            fn = registry.resolve_operator(name, "generic_module_that_is_never_imported", generic, vendor="amd")
            out[name] = [fn.__module__, fn.__qualname__]
        # an operator the package does not declare keeps the generic implementation
        fn = registry.resolve_operator("flash_attention", "math", "sqrt", vendor="amd")
        out["flash_attention (not declared: generic math.sqrt)"] = [fn.__module__, fn.__qualname__]
        return out
    finally:
        if saved is None:
            sys.modules.pop(BACKEND_NAME, None)
        else:
            sys.modules[BACKEND_NAME] = saved


if __name__ == "__main__":
    result = resolve_with_reference_registry()
    with open(os.path.join(HERE, "registry_golden.json"), "w") as f:
        json.dump(result, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(result, indent=1))
