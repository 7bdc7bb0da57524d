"""Rules the kernel sources keep that no GPU test can be relied on to catch.

gfx940-family parts change what a store of more than 64 bits writes when a VALU instruction overwrites the
store's data registers within two wait states of it.  The compiler spaces its own stores, but it cannot know that
an ``asm`` statement is a store: every 128-bit store issued through inline asm therefore has to bring its own two
wait states (``s_nop 1``).  Whether the hazard bites depends on the register allocation of one build, so a parity
test may pass for years with the rule broken.
"""
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "rannc_amd", "csrc")


def _asm_statements(text):
    text = re.sub(r"^\s*#define\s+(\w+)\s+(\"[^\n]*\")\s*$", "", text, flags=re.M)
    return re.findall(r"asm\s+volatile\s*\((.*?)\)\s*;", text, flags=re.S)


def test_every_128_bit_asm_store_waits_two_states():
    seen = 0
    for path in sorted(glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(CSRC, "*.hip"))):
        text = open(path).read()
        macros = dict(re.findall(r"^\s*#define\s+(\w+)\s+\"((?:[^\"\\]|\\.)*)\"\s*$", text, flags=re.M))
        for stmt in _asm_statements(text):
            if "global_store_dwordx4" not in stmt and "global_store_dwordx3" not in stmt:
                continue
            seen += 1
            template = stmt.split(":")[0]
            for name, value in macros.items():
                template = template.replace(name, '"' + value + '"')
            assert "s_nop 1" in template, f"{os.path.basename(path)}: 128-bit asm store without its wait states: {stmt.strip()[:120]}"
    assert seen >= 1, "expected to find the asm store the header keeps for comparison builds"
