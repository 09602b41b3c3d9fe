"""The ctypes mirrors of the C ABI's structures (splitrpc_amd/capi.py) against
include/sg_hip.h as a C compiler lays it out: every field by name, offset and
size.  No GPU needed."""
import ctypes as C
import os
import subprocess

from splitrpc_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

MIRRORS = [("sg_hbufs", capi.HBufs), ("sg_sk_buf", capi.SkBuf), ("sg_hip_cfg", capi.Cfg),
           ("sg_ring_desc", capi.RingDesc), ("sg_app_desc", capi.AppDesc), ("sg_gather_args", capi.GatherArgs),
           ("sg_scatter_args", capi.ScatterArgs), ("sg_reassemble_args", capi.ReassembleArgs),
           ("sg_frag_table", capi.FragTable), ("sg_pack_args", capi.PackArgs)]


def test_ctypes_mirrors_match_the_header(tmp_path):
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "sg_hip.h"', 'int main(void) {']
    want = []
    for cname, mirror in MIRRORS:
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        want.append(f"{cname} {C.sizeof(mirror)}")
        for fname, _ in mirror._fields_:
            lines.append(f'  printf("{cname}.{fname} %zu %zu\\n", offsetof({cname}, {fname}), '
                         f'sizeof((({cname} *)0)->{fname}));')
            f = getattr(mirror, fname)
            want.append(f"{cname}.{fname} {f.offset} {f.size}")
    for name in ("SG_MAX_BI_SIZE", "SG_MAX_TENSORS", "SG_HIP_ABI_VERSION", "SG_STATIC_MAX_REQS",
                 "SG_STATIC_MAX_FRAMES"):
        lines.append(f'  printf("{name} %ld\\n", (long)({name}));')
    want += [f"SG_MAX_BI_SIZE {capi.MAX_BI_SIZE}", f"SG_MAX_TENSORS {capi.MAX_TENSORS}",
             f"SG_HIP_ABI_VERSION {capi.ABI_VERSION}", f"SG_STATIC_MAX_REQS {capi.STATIC_MAX_REQS}",
             f"SG_STATIC_MAX_FRAMES {capi.STATIC_MAX_FRAMES}"]
    for name in ("SG_F_IPV4_CSUM", "SG_F_UDP_CSUM_FULL", "SG_F_UDP_CSUM_PSEUDO", "SG_F_REF_QUIRKS", "SG_F_RULE_FRAGS",
                 "SG_F_NO_FUSE", "SG_F_REUSE_DESC", "SG_F_ASYNC", "SG_F_NO_XCD_REMAP", "SG_F_NO_SMALL", "SG_F_FORCE_SMALL"):
        lines.append(f'  printf("{name} %ld\\n", (long)({name}));')
        want.append(f"{name} {getattr(capi, name[3:])}")
    lines += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)],
                   check=True)
    got = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.strip().splitlines()
    assert got == want
