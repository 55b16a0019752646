"""The split row reduction publishes a block's accumulator and then counts the block in on a
ticket; the block that counts in last reads every accumulator. The ticket add is relaxed (a
release at agent scope writes back the die's whole second-level cache, once per block), so
what orders the publication before the count is the instruction sequence itself:

    global_store_dword ... sc1          the accumulator, written through at agent scope
    s_waitcnt vmcnt(0) ...              its acknowledgement
    global_atomic_add ...               the ticket

and, in the block that counted in last, `buffer_inv sc1` (the acquire) before the first load
of an accumulator. This test compiles one instance of the kernel to assembly (device side
only, about a second) and checks that sequence, so that a compiler that reorders it fails
here and not as a rare wrong sum."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

pytestmark = pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is not present")


def split_kernel_asm(tmp_path):
    out = tmp_path / "ordering_probe.s"
    cmd = [HIPCC, "-O3", "-std=c++17", "-ffp-contract=off", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "cumo_amd", "csrc"),
           "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only", "-x", "hip",
           os.path.join(ROOT, "tests", "ordering_probe.hip"), "-o", str(out)]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=str(tmp_path))
    assert p.returncode == 0, p.stdout[-2000:]
    text = out.read_text()
    m = re.search(r"^_ZN8cumo_hip21red_srow_split_kernel\w*:[^\n]*\n(.*?)\n\s*s_endpgm", text, flags=re.S | re.M)
    assert m, "the split kernel is not in the assembly"
    return [l.strip() for l in m.group(1).splitlines() if l.strip() and not l.strip().startswith(";")]


def test_publication_is_acknowledged_before_the_ticket(tmp_path):
    lines = split_kernel_asm(tmp_path)
    ops = [(i, l) for i, l in enumerate(lines) if re.match(r"(global_store|global_atomic|s_waitcnt|buffer_inv|buffer_wbl2|global_load)", l)]
    publish = [i for i, l in ops if l.startswith("global_store_dword") and "sc1" in l]
    tickets = [i for i, l in ops if l.startswith("global_atomic_add")]
    assert publish and len(tickets) == 2, (publish, tickets)
    first_publish, first_ticket = publish[0], tickets[0]
    assert first_publish < first_ticket, "the accumulator must be stored before the block counts in"
    # between them: a wait for ALL outstanding vector memory operations, and nothing that writes back the cache
    between = [l for i, l in ops if first_publish < i < first_ticket]
    assert any(re.match(r"s_waitcnt\b.*vmcnt\(0\)", l) for l in between), between
    assert not any(l.startswith("buffer_wbl2") for l in lines), "a cache write-back per block costs four times the kernel's run time"
    # no store of the accumulator after the first ticket (the publication is complete by then):
    # the stores that follow the tickets are the ones that put a ticket back to zero
    acc_stores_after = [l for i, l in ops if i > first_ticket and l.startswith("global_store_dword") and "sc1" in l]
    assert len(acc_stores_after) == 2, acc_stores_after
    # the last block acquires before it reads the others' accumulators
    inv = [i for i, l in ops if l.startswith("buffer_inv") and "sc1" in l]
    assert inv and inv[0] > tickets[-1], (inv, tickets)
    loads_after_inv = [l for i, l in ops if i > inv[0] and l.startswith("global_load")]
    loads_between = [l for i, l in ops if tickets[-1] < i < inv[0] and l.startswith("global_load")]
    assert loads_after_inv and not loads_between, "accumulators may only be read after the acquire"
