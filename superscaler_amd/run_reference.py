"""Run one of the reference's search scripts over this library, leaving the reference's tree as it is:

    cd <reference>/search
    python -m superscaler_amd.run_reference aceso_search.py --model-name gpt --model-size 1_3B ...    (the script's own flags)
    python -m superscaler_amd.run_reference gen_megatron_plan.py ...

The scripts do `from aceso_cost_model import ...` (aceso_search.py:4, aceso_prims.py:7, gen_megatron_plan.py:8).  This
launcher puts the script's directory on sys.path, registers the binding file (superscaler_amd/binding/aceso_cost_model.py)
under the module name `aceso_cost_model` before anything imports it, and then runs the script as `__main__` with the
remaining arguments: the same effect as copying the binding file over search/aceso_cost_model.py.  The reference's
import-time parse_args() (aceso_cost_model.py:10) runs inside the binding on those arguments.  aceso_search.py forks one
process per stage count; the children inherit the registered module and create their GPU handles after the fork."""
import importlib.util
import os
import runpy
import sys


def install_binding(search_dir: str):
    """Register the binding as module `aceso_cost_model` (sys.argv must already hold the reference's flags: its
    parse_args() runs now).  Returns the module."""
    search_dir = os.path.abspath(search_dir)
    if search_dir not in sys.path:
        sys.path.insert(0, search_dir)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "binding", "aceso_cost_model.py")
    spec = importlib.util.spec_from_file_location("aceso_cost_model", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["aceso_cost_model"] = mod
    try:
        spec.loader.exec_module(mod)
    except BaseException:
        del sys.modules["aceso_cost_model"]
        raise
    return mod


def main(argv=None) -> int:
    argv = sys.argv[1:] if argv is None else list(argv)
    if not argv or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 2
    script = os.path.abspath(argv[0])
    if not os.path.isfile(script):
        print(f"no such script: {argv[0]}", file=sys.stderr)
        return 2
    sys.argv = [script] + argv[1:]
    install_binding(os.path.dirname(script))
    runpy.run_path(script, run_name="__main__")
    return 0


if __name__ == "__main__":
    sys.exit(main())
