"""The front end run over the reference's own complete input -> output examples.

Fifty directories of the reference hold the fuser's input (`cuda/kernels.cu`, TVM-generated
CUDA), its configuration and what the reference's Clang-based fuser emitted for it
(`cuda/bfuse_kernels.cu`, `cuda/hfuse_kernels.cu`): legacy/tests/single_bgemm_conv2d/case-*/
{M,N}_diff/case-*/ and legacy/tests/block_scheduler_test/.  They are read in place, as text
(nothing of them is stored here), so this file only runs where the reference tree is mounted
and is skipped elsewhere.  For every directory the front end is run on the same input with
the options that directory was generated with, and

  * the dispatch chain it prints evaluates, on sampled block ids, to what the reference's
    printed chain evaluates to;
  * the two rewritten kernel bodies equal the reference's character for character once
    whitespace, comments and the spelling of float literals (Clang's printer writes `0.F`)
    are normalised;
  * for thread-level fusion the same holds after the reference's `bar.sync id, count` lines
    and this tool's side barriers are both reduced to (side, threads) markers.
"""
import glob
import json
import os
import random
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FUSER = os.path.join(ROOT, "bfuse-project_amd", "horizontal-fuser")
REF = os.environ.get("BFUSE_REFERENCE", "/root/reference")
TRIOS = sorted(os.path.dirname(os.path.dirname(p)) for p in glob.glob(os.path.join(REF, "legacy/tests/**/cuda/bfuse_kernels.cu"), recursive=True)
               if os.path.exists(os.path.join(os.path.dirname(p), "kernels.cu")) and os.path.exists(os.path.join(os.path.dirname(p), "hfuse_kernels.cu")))

pytestmark = pytest.mark.skipif(not TRIOS or not os.path.exists(FUSER), reason="reference tree or front end not present")


def options_of(trio):
    """The pattern options a directory was generated with, from the fixture that records them."""
    rel = os.path.relpath(os.path.join(trio, "cuda", "bfuse_kernels.cu"), REF)
    for e in json.load(open(os.path.join(ROOT, "tests", "golden", "bfuse_maps.json"))):
        if e["source"] == rel:
            if e["pattern"] == "zigzag":
                return ["-M", str(e["params"]["M"]), "-N", str(e["params"]["N"])], e
            return ["-p", "chunked", "-c", str(e["params"]["TotalSM"])], e
    return None, None


def norm(text):
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"(?<![\w.])(\d+\.\d*(?:[eE][+-]?\d+)?|\d+[eE][+-]?\d+)[fF]\b", lambda m: f"<{float(m.group(1))!r}>", text)
    text = text.replace("__restrict__", "__restrict")      # Clang's printer drops the trailing underscores
    return re.sub(r"\s+", "", text)


def c_to_py(expr):
    expr = expr.replace("(int)blockIdx.x", "b").replace("&&", " and ").replace("||", " or ")
    return re.sub(r"\bint\(", "(", expr).replace("/", "//")


def chain_of(text):
    chain = re.findall(r"if \((.*)\)\s*\{\s*NewBlockIdx_ = (.*);\s*KernelID_\s*= (\d+);", text)
    assert chain
    return [(c_to_py(c), c_to_py(v), int(k)) for c, v, k in chain]


def eval_chain(chain, bid):
    for cond, virt, kid in chain:
        if eval(cond, {"b": bid}):
            return kid, eval(virt, {"b": bid})
    return -1, -1


def fuse(trio, tmp_path, *opts):
    cfg = os.path.join(trio, "config")
    out = tmp_path / "out"
    r = subprocess.run([FUSER, *opts, "-o", str(out), "-y", str(out), os.path.join(cfg, "fusions.yaml"),
                        os.path.join(cfg, "kernels.yaml"), os.path.join(trio, "cuda")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    return out


def test_there_are_fifty():
    assert len(TRIOS) == 50


@pytest.mark.parametrize("trio", TRIOS, ids=[os.path.relpath(t, REF) for t in TRIOS])
def test_block_fusion_output_equals_reference(trio, tmp_path):
    opts, entry = options_of(trio)
    if opts is None:
        pytest.skip("options of this directory are not recorded")
    out = fuse(trio, tmp_path, "-b", *opts)
    ref = open(os.path.join(trio, "cuda", "bfuse_kernels.cu")).read()
    mine = open(glob.glob(str(out / "*_bfuse.hip"))[0]).read()
    # same dispatch
    rc, mc = chain_of(ref), chain_of(mine)
    rng = random.Random(7)
    total = entry["fused_grid"]
    bids = sorted(set(list(range(0, min(total, 600))) + [rng.randrange(total) for _ in range(400)] + list(range(max(0, total - 300), total + 2))))
    for b in bids:
        assert eval_chain(mc, b) == eval_chain(rc, b), b
    # same bodies (everything after the LDS union object)
    tail_ref, tail_mine = norm(ref[ref.index("SU_;"):]), norm(mine[mine.index("SU_;"):])
    if "streamingMultiprocessorId" in tail_ref:
        # block_scheduler_test: its input carries a hand-written %smid probe in both kernels, which
        # the checked-in output has in one, hand-moved, place; the output also has an older
        # spelling of the thread guard (`tid >= 0 && tid < T`)
        probe = r'uintstreamingMultiprocessorId;asm\(.*?\);printf\(.*?\);'
        tail_ref, tail_mine = re.sub(probe, "", tail_ref), re.sub(probe, "", tail_mine)
        tail_ref = re.sub(r"\(\(int\)threadIdx\.x>=0&&\(int\)threadIdx\.x<(\d+)\)", r"((int)threadIdx.x<\1)", tail_ref)
    assert tail_mine == tail_ref
    # same signature and LDS union members
    sig = lambda t: norm(t[t.index("__launch_bounds__"):t.index("{")])
    assert sig(mine) == sig(ref)
    union = lambda t: norm(t[t.index("typedef union"):t.index("SU_;")]) if "typedef union" in t else norm(t[t.index("union"):t.index("SU_;")])
    assert union(mine) == union(ref)


def _hfuse_markers(text, mine):
    if mine:
        # side barrier call -> <bar side waves*64>
        text = re.sub(r"bfuse_side_barrier\(&bfuse_arrive_\[(\d+)\], (\d+)u, &bfuse_epoch_\);", lambda m: f"<bar {int(m.group(1))} >;", text)
    else:
        text = re.sub(r'asm\s*(?:volatile)?\s*\(\s*"bar\.sync (\d+), (\d+);"\s*\);', lambda m: f"<bar {int(m.group(1)) - 1} >;", text)
    return text


@pytest.mark.parametrize("trio", TRIOS, ids=[os.path.relpath(t, REF) for t in TRIOS])
def test_thread_fusion_bodies_equal_reference(trio, tmp_path):
    out = fuse(trio, tmp_path, "-w", "32")
    ref = open(os.path.join(trio, "cuda", "hfuse_kernels.cu")).read()
    mine = open(glob.glob(str(out / "*_hfuse.hip"))[0]).read()
    # the statements of each side after its remap declarations: from the first statement that
    # is not a declaration of an index variable to the end of the branch
    def sides(text, is_mine):
        text = _hfuse_markers(text, is_mine)
        parts = re.split(r"if \(\(\(int\)threadIdx\.x >= \d+ && \(int\)threadIdx\.x < \d+\)", text)[1:]
        res = []
        for p in parts:
            body = p[p.index("{") + 1:]
            # drop index declarations, (void) casts and this tool's epoch variable
            body = re.sub(r"(?:unsigned )?int (?:blockIdx|threadIdx|gridDim|blockDim)_[xyz]_[^;]*;", "", body)
            body = re.sub(r"\(void\)\w+;", "", body)
            body = re.sub(r"unsigned int bfuse_epoch_ = 0u;", "", body)
            body = re.sub(r"static\s+(\w[\w\s]*?)\s+(\w+)(\[[^\]]*\])?\s*__attribute__\(\(shared\)\)", r"__shared__ \1 \2\3", body)
            res.append(norm(body))
        return res
    sr, sm = sides(ref, False), sides(mine, True)
    assert len(sr) == len(sm) == 2
    # block_scheduler_test carries a hand-placed %smid probe (in its input and, moved, in its outputs)
    probe = lambda t: re.sub(r'uintstreamingMultiprocessorId;asm\(.*?\);printf\(.*?\);', "", t)
    for a, b in zip(sr, sm):
        # both end with the closing braces of the branch and of the kernel
        assert probe(a).rstrip("}") == probe(b).rstrip("}")


def test_emitted_code_compiles_for_gfx950(tmp_path):
    trio = min(TRIOS, key=lambda t: os.path.getsize(os.path.join(t, "cuda", "kernels.cu")))
    opts, _ = options_of(trio)
    out = fuse(trio, tmp_path, "-b", *(opts or []))
    fuse(trio, tmp_path, )
    for f in sorted(glob.glob(str(out / "*.hip"))):
        r = subprocess.run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "--genco", "-O1", f, "-o", f[:-4] + ".hsaco"],
                           capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
