"""The generated gfx950 code of every kernel, checked without a GPU: the sources are compiled to
assembly (hipcc cross-compiles here) and the text is searched for what must not be there.

* no flat loads or stores (table-derived addresses must stay in the global address space),
* no scratch memory (no register spills in a streaming kernel),
* no packed fp32 arithmetic (the build switches its formation off),
* no loop that makes a buffer resource uniform lane by lane (the windows' bases are uniform),
* every 16-byte load of streamed data carries the non-temporal hint -- the compiler drops it
  silently from a vector load that is only byte-aligned, which is why byte elements are read
  through raw buffer loads -- except in the Adasum first pass, which keeps one or both of its
  vectors cached on purpose."""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "horovod_amd", "csrc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-mllvm", "-amdgpu-kernarg-preload-count=16", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
         "-S", "--cuda-device-only"]


def _assembly(tmp, name):
    out = os.path.join(tmp, name + ".s")
    r = subprocess.run(["hipcc"] + FLAGS + ["-o", out, os.path.join(CSRC, name + ".hip")],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=600)
    assert r.returncode == 0, r.stdout.decode(errors="replace")[-2000:]
    return open(out).read()


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    """{kernel symbol: [instruction lines]} over the three kernel sources."""
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc is not installed")
    tmp = str(tmp_path_factory.mktemp("isa"))
    with ThreadPoolExecutor(3) as pool:
        texts = list(pool.map(lambda n: _assembly(tmp, n), ["xfer", "reduce", "adasum"]))
    found = {}
    for text in texts:
        name = None
        for line in text.splitlines():
            m = re.match(r"^(_ZN6hvdhip\S+):\s*; @", line)
            if m:
                name = m.group(1)
                found[name] = []
            elif name and line.startswith("\t") and not line.lstrip().startswith((";", ".")):
                found[name].append(line.strip())
                if line.strip().startswith("s_endpgm"):
                    name = None
    assert len(found) > 200, len(found)  # every instantiation of the three kernel families
    return found


def test_no_flat_scratch_or_packed_fp32(kernels):
    for name, lines in kernels.items():
        for ins in lines:
            op = ins.split()[0]
            # a buffer resource that the compiler cannot prove uniform is made uniform in a loop
            assert not op.startswith("v_readfirstlane"), (name, ins)
            assert not op.startswith(("flat_load", "flat_store")), (name, ins)
            assert not op.startswith("scratch_"), (name, ins)
            assert not re.match(r"v_pk_\w+_f32", op), (name, ins)


def test_streaming_loads_keep_the_non_temporal_hint(kernels):
    checked = 0
    for name, lines in kernels.items():
        if "finalize_k" in name:
            continue  # reads the small table of partial sums, nothing streamed
        # the Adasum first pass leaves a (mode 1) or a and b (mode 2) in the Infinity Cache on purpose
        m = re.search(r"dot_partials_kI\w+?Li([12])EEE", name)
        keeps = m is not None and m.group(1) == "2"
        keeps_a = m is not None and m.group(1) == "1"
        # the fused scaled add also reads its layer's partial sums (24 bytes each, two per lane): not streamed
        fused = re.search(r"scaled_add_kI\w+?Lb1ELi[01]EEE", name) is not None
        plain = hinted = 0
        for ins in lines:
            op = ins.split()[0]
            if op in ("global_load_dwordx4", "buffer_load_dwordx4"):
                checked += 1
                if keeps:
                    assert " nt" not in ins, (name, ins)
                elif " nt" not in ins:
                    plain += 1
                else:
                    hinted += 1
        if keeps_a:
            assert plain == hinted and plain > 0, (name, plain, hinted)  # a plainly, b with the hint
        else:
            assert plain <= (4 if fused else 0), (name, plain)
    assert checked > 500, checked


def test_streaming_stores_carry_one_of_the_two_policies(kernels):
    """Vector stores of streamed data are non-temporal global stores or write-through buffer
    stores (sc0 sc1); a plain store would leave its lines in L2 for neither reader."""
    checked = 0
    for name, lines in kernels.items():
        if "finalize_k" in name or "one_layer_tables_k" in name:
            continue  # stores a layer's sums and coefficients, or a chunk table: nothing streamed
        # sums and coefficients of a layer or chunk, written by one lane
        small_results = 4 if ("scaled_add_k" in name or "dot_partials_k" in name) else 0
        plain = 0
        for ins in lines:
            op = ins.split()[0]
            if op == "global_store_dwordx4":
                checked += 1
                plain += " nt" not in ins
            elif op in ("buffer_store_dwordx4", "buffer_store_dwordx2"):
                checked += 1
                assert " sc0 sc1" in ins and " nt" not in ins, (name, ins)
        assert plain <= small_results, (name, plain)
    assert checked > 500, checked


def test_scaled_add_products_are_not_fused_into_the_sum(kernels):
    """ScaledAdd (ops/adasum/adasum.h:429-435) is two rounded double products and their rounded
    sum.  In the kernels that take their coefficients ready-made the only double arithmetic is
    that expression, so a fused multiply-add there would be a contracted product."""
    checked = 0
    for name, lines in kernels.items():
        m = re.search(r"scaled_add_kI([fd])Lb0ELi[01]EEE", name)
        if not m:
            continue
        ops = [ins.split()[0] for ins in lines]
        assert not any(op.startswith(("v_fma_f64", "v_fmac_f64")) for op in ops), name
        muls = sum(op.startswith("v_mul_f64") for op in ops)
        adds = sum(op.startswith("v_add_f64") for op in ops)
        assert muls == 2 * adds and adds > 0, (name, muls, adds)
        checked += 1
    assert checked == 4


def test_contiguous_kernels_reach_their_first_load_without_a_scalar_branch(kernels):
    """A workgroup of the reduce-sum or the whole-buffer scale computes its tile number without
    branching and fetches the arguments that were not preloaded in one go: a chain of dependent
    scalar loads and branches ahead of the first data load is paid in full by a grid that the
    device holds all at once (the 7-peer sum of an 8 MiB chunk: 14.5 against 12.6 us)."""
    checked = 0
    for name, lines in kernels.items():
        if "reduce_k" not in name and "contig_k" not in name:
            continue
        ops = [ins.split()[0] for ins in lines]
        first = next(i for i, op in enumerate(ops) if op.startswith(("global_load", "buffer_load")))
        head = ops[:first]
        assert not any(op.startswith("s_cbranch_scc") for op in head), name
        # the compatibility prologue for firmware that does not preload waits once, the kernel proper at most once
        assert sum(op == "s_waitcnt" for op in head) <= 2, (name, head)
        checked += 1
    assert checked >= 100, checked
