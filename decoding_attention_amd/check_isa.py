"""Build-time check of da_mla_pipe.hip's generated code.

That kernel names most of the register file in its instruction text (Q in v112..v255, the output tiles in a0..a255,
the LDS fragment ring in v80..v111, the probability tile in v64..v79) and confines the compiler's own allocation to v0..v63 with a kernel attribute.
Nothing tells the compiler that the named registers hold live values, so the build verifies what it generated:
outside the hand-written instruction blocks there must be no vector register above v63, no accumulation register
and no scratch access.  A violation would corrupt the kernel's state silently, so it fails the build.
"""
import re
import subprocess
import sys

COMPILER_VGPR_LIMIT = 64


def check_text(asm_text, limit=COMPILER_VGPR_LIMIT):
    """Return a list of violations (line number, text) in the assembly text of one translation unit."""
    bad = []
    in_asm = False
    for i, line in enumerate(asm_text.split("\n"), 1):
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        s = line.strip()
        if in_asm or not s or s.startswith(";") or s.startswith(".") or s.endswith(":"):
            continue
        s = s.split(";")[0]
        top = -1
        for m in re.finditer(r"\bv(\d+)\b", s):
            top = max(top, int(m.group(1)))
        for m in re.finditer(r"\bv\[(\d+):(\d+)\]", s):
            top = max(top, int(m.group(2)))
        if top >= limit:
            bad.append((i, line))
        elif "accvgpr" in s or re.search(r"\ba\d+\b|\ba\[\d+", s):
            bad.append((i, line))
        elif "scratch_" in s:
            bad.append((i, line))
    return bad


def check_source(hipcc, flags, src):
    """Compile `src` to device assembly with the given flags and check it; raises on a violation."""
    cmd = [hipcc] + flags + ["-S", "--cuda-device-only", "-o", "-", src]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src}:\n{res.stderr}")
    if "latent_pipe_kernel" not in res.stdout:
        raise RuntimeError(f"{src}: no latent_pipe_kernel in the generated assembly")
    bad = check_text(res.stdout)
    if bad:
        shown = "\n".join(f"  line {i}: {t.strip()}" for i, t in bad[:10])
        raise RuntimeError(f"{src}: the compiler left its register range in {len(bad)} places "
                           f"(it must stay below v{COMPILER_VGPR_LIMIT}, off the accumulation registers and off "
                           f"scratch):\n{shown}")
    return True


if __name__ == "__main__":
    text = open(sys.argv[1]).read()
    v = check_text(text)
    for i, t in v[:20]:
        print(f"line {i}: {t.strip()}")
    print("violations:", len(v))
    sys.exit(1 if v else 0)
