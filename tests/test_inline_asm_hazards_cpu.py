"""The global->LDS tile loads are issued from inline assembly (``moda_amd/csrc/tile.h: lds_dma``), which the
compiler's hazard pass does not look into.  On gfx9-family hardware a vector-memory instruction that reads a
scalar register written by a vector-ALU instruction (``v_readfirstlane_b32``, ``v_readlane_b32`` restoring a
spilled scalar, ...) fewer than five wait states earlier sees the register's old value -- for a tile load that is
a stale descriptor base, size or offset.  The compiler does place such writes directly in front of the assembly
block when scalar registers are short (dozens of sites in the forward kernels), so the block carries its own wait
states.  This test compiles the three matrix kernels' sources to assembly (device pass only, no GPU needed) and
checks every tile load: at least five wait states since the last vector-ALU write of any scalar register it reads.
"""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "moda_amd", "csrc")
NEED = 5
VALU_SGPR_WRITERS = re.compile(r"(v_readlane_b32|v_readfirstlane_b32|v_cmp\w*|v_cmpx\w*|v_add_co\w*|v_sub_co\w*|v_subrev_co\w*|"
                               r"v_addc_co\w*|v_subb_co\w*|v_div_scale\w*|v_mad_u64_u32|v_mad_i64_i32)\s+(.*)")


def sregs(tok):
    tok = tok.strip().rstrip(",")
    m = re.fullmatch(r"s\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"s(\d+)", tok)
    return {int(m.group(1))} if m else set()


def written_sgprs(ins):
    m = VALU_SGPR_WRITERS.match(ins)
    if not m:
        return set()
    ops = [o.strip() for o in m.group(2).split(",")]
    out = set()
    # the scalar destination is the first operand, or the second one of the carry-out / 64-bit multiply-add forms
    for o in ops[:2]:
        out |= sregs(o)
    return out


def wait_states(ins):
    m = re.match(r"s_nop (\d+)", ins)
    return int(m.group(1)) + 1 if m else 1


def scan(path):
    window, sites, bad = [], 0, []
    for ln, raw in enumerate(open(path), 1):
        line = raw.split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        if "buffer_load_dword" in line and line.endswith("lds"):
            sites += 1
            used = set()
            for t in line.split(None, 1)[1].replace("offen", "").replace("lds", "").split(","):
                used |= sregs(t)
            ws = 0
            for ins in reversed(window):
                if ws >= NEED:
                    break
                if written_sgprs(ins) & used:
                    bad.append((ln, ins, line, ws))
                ws += wait_states(ins)
        window.append(line)
        if len(window) > 16:
            window.pop(0)
    return sites, bad


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not found")
    out = tmp_path_factory.mktemp("asm")

    def build(name):
        dst = str(out / (name + ".s"))
        subprocess.run(["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                        "-packed-fp32-ops", "--cuda-device-only", "-S", os.path.join(CSRC, name + ".hip"), "-o", dst],
                       check=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
        return dst

    with ThreadPoolExecutor(4) as ex:
        return list(ex.map(build, ["fwd_kernel", "bwd_dq_kernel", "bwd_dkv_kernel", "bwd_dkv_flat_kernel"]))


def test_scanner_sees_the_hazard():
    import tempfile

    text = """
\tv_readfirstlane_b32 s4, v66
\ts_mov_b32 m0, s20
\ts_nop 0
\tbuffer_load_dwordx4 v141, s[4:7], s10 offen lds
\tv_readlane_b32 s10, v254, 3
\ts_mov_b32 m0, s20
\ts_nop 3
\tbuffer_load_dwordx4 v141, s[4:7], s10 offen lds
"""
    with tempfile.NamedTemporaryFile("w", suffix=".s", delete=False) as f:
        f.write(text)
    sites, bad = scan(f.name)
    os.unlink(f.name)
    assert sites == 2 and len(bad) == 1 and bad[0][3] == 2


def test_tile_loads_keep_five_wait_states_after_vector_writes_of_their_scalars(assembly):
    total = 0
    for path in assembly:
        sites, bad = scan(path)
        total += sites
        assert not bad, f"{os.path.basename(path)}: {len(bad)} tile loads too close to a vector-ALU scalar write, e.g. {bad[:3]}"
    assert total > 1000  # the scan did find the loads (every instantiation of the four kernel files)
