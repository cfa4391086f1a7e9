"""The assembly op loop is committed as generated text (superscaler_amd/csrc/ace_score_loop_asm.inc): it must be what
its generator writes today, or an edit of one of the two was not carried to the other."""
import importlib.util
import os

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "superscaler_amd", "csrc")


def _generator():
    spec = importlib.util.spec_from_file_location("gen_score_loop_asm", os.path.join(CSRC, "gen_score_loop_asm.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_committed_loop_text_is_the_generators_output():
    with open(os.path.join(CSRC, "ace_score_loop_asm.inc")) as f:
        committed = f.read()
    assert committed == _generator().render()


def test_every_loop_variant_is_defined_and_owns_only_its_registers():
    """One text per (rows resident / windowed, resharding, reserved-memory rule); no text names a vector register below
    v28 or a scalar register below s24 (those hold the statement's operands) or the stack registers s32 / s33."""
    import re
    text = _generator().render()
    names = re.findall(r"#define (ACE_LOOP_ASM\w*) ", text)
    want = {f"ACE_LOOP_ASM{w}_RSH{r}_{m}" for w in ("", "_WIN") for r in (0, 1) for m in ("MAX", "MIN", "NONE")} | {"ACE_LOOP_ASM_CLOBBERS"}
    assert set(names) == want
    body = text.split("#define ACE_LOOP_ASM_CLOBBERS")[0]
    for m in re.finditer(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]", body):
        lo = int(m.group(1) or m.group(2))
        hi = int(m.group(1) or m.group(3))
        assert 28 <= lo <= hi <= 127, m.group(0)
    for m in re.finditer(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]", body):
        lo = int(m.group(1) or m.group(2))
        hi = int(m.group(1) or m.group(3))
        assert 24 <= lo <= hi <= 99 and not (lo <= 33 and hi >= 32), m.group(0)
