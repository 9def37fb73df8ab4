"""Config wire format of the fuser: kernels.yaml / fusions.yaml / {b,h}fuse_kernels.yaml.

Schema of the reference's llvm::yaml traits (horizontal-fuser/include/fuse/Utils.h:70-112)
and data model (horizontal-fuser/include/fuse/Contexts.h:13-106).  Files written by the
reference's tools load unchanged, and files written here load in the reference.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import yaml

from .patterns import LaunchDims, plan_blocks, plan_threads


@dataclass
class KernelInfo:
    """Contexts.h:28-51.  Reg and HasBarriers are parsed but unused by the reference's
    patterns; here `choose_fusion` consumes them."""
    KernelName: str
    HasBarriers: bool
    GridDim: Tuple[int, int, int]
    BlockDim: Tuple[int, int, int]
    Reg: int
    ExecTime: float = -1.0

    @property
    def dims(self) -> LaunchDims:
        return LaunchDims(tuple(self.GridDim), tuple(self.BlockDim))

    def to_yaml_dict(self):
        d = {"KernelName": self.KernelName, "HasBarriers": bool(self.HasBarriers),
             "GridDim": dict(zip("XYZ", self.GridDim)), "BlockDim": dict(zip("XYZ", self.BlockDim)),
             "Reg": int(self.Reg)}
        if self.ExecTime != -1:
            d["ExecTime"] = float(self.ExecTime)
        return d


@dataclass
class FusionInfo:
    """Contexts.h:53-62."""
    File: str
    Kernels: List[str] = field(default_factory=list)


def _xyz(d, what, name):
    try:
        return int(d["X"]), int(d["Y"]), int(d["Z"])
    except (KeyError, TypeError) as e:
        raise ValueError(f"{name}: {what} needs integer X, Y, Z") from e


def parse_kernels(doc) -> Dict[str, KernelInfo]:
    if not isinstance(doc, dict):
        raise ValueError("kernels.yaml must be a mapping of name -> KernelInfo")
    out = {}
    for name, e in doc.items():
        for req in ("KernelName", "HasBarriers", "GridDim", "BlockDim", "Reg"):   # mapRequired, Utils.h:75-79
            if not isinstance(e, dict) or req not in e:
                raise ValueError(f"{name}: missing required key {req}")
        out[str(name)] = KernelInfo(str(e["KernelName"]), bool(e["HasBarriers"]), _xyz(e["GridDim"], "GridDim", name),
                                    _xyz(e["BlockDim"], "BlockDim", name), int(e["Reg"]),
                                    float(e.get("ExecTime", -1)))                 # mapOptional, Utils.h:80
    return out


def parse_fusions(doc) -> List[FusionInfo]:
    if not isinstance(doc, list):
        raise ValueError("fusions.yaml must be a sequence of {File, Kernels}")
    out = []
    for e in doc:
        if not isinstance(e, dict) or "File" not in e or "Kernels" not in e:
            raise ValueError("fusion entry needs File and Kernels")
        out.append(FusionInfo(str(e["File"]), [str(k) for k in e["Kernels"]]))
    return out


def load_kernels_yaml(path) -> Dict[str, KernelInfo]:
    with open(path) as f:
        return parse_kernels(yaml.safe_load(f))


def load_fusions_yaml(path) -> List[FusionInfo]:
    with open(path) as f:
        return parse_fusions(yaml.safe_load(f))


def dump_kernels_yaml(infos: Dict[str, KernelInfo], path=None) -> str:
    text = yaml.safe_dump({k: v.to_yaml_dict() for k, v in infos.items()}, sort_keys=False)
    if path:
        with open(path, "w") as f:
            f.write(text)
    return text


# per-CU limits of gfx950 that bound how two sides share a CU
LDS_PER_CU = 160 * 1024
VGPRS_PER_SIMD = 512
MAX_WAVES_PER_SIMD = 8


@dataclass
class FusionContext:
    """FusionContext::create (horizontal-fuser/src/Contexts.cc:56-92): fused name
    `<K1>_<K2>_fused_{bfuse,hfuse}` and fused launch shape from the selected pattern."""
    Kernels: List[str]
    FusedKernelName: str
    FusedGridDim: Tuple[int, int, int]
    FusedBlockDim: Tuple[int, int, int]
    plan: object

    @staticmethod
    def create(finfo: FusionInfo, kmap: Dict[str, KernelInfo], bfuse: bool, pattern: str = "zigzag",
               p0: int = 1, p1: int = 1, pad: int = 64) -> "FusionContext":
        infos = [kmap[k] for k in finfo.Kernels]      # KeyError on an unknown kernel, like map::at (Contexts.cc:69)
        name = "".join(k + "_" for k in finfo.Kernels) + ("fused_bfuse" if bfuse else "fused_hfuse")
        dims = [i.dims for i in infos]
        plan = plan_blocks(pattern, dims, p0, p1) if bfuse else plan_threads(dims, pad)
        return FusionContext(list(finfo.Kernels), name, (plan.fused_grid, 1, 1), (plan.fused_block, 1, 1), plan)

    def fused_kernel_info(self) -> KernelInfo:
        # the reference records Reg = 32, HasBarriers = true for every fused kernel (Fuse.cc:204-209)
        return KernelInfo(self.FusedKernelName, True, self.FusedGridDim, self.FusedBlockDim, 32)


def choose_fusion(a: KernelInfo, b: KernelInfo, lds_a: int, lds_b: int, cus: int = 256, matrix=(False, False)) -> dict:
    """Picks hfuse vs bfuse vs no fusion from each side's footprint (and its ExecTime where known).

    * Both sides with barriers -> block fusion (a wave-granular LDS barrier on both sides of
      one workgroup would have each side spin on issue slots the other needs).
    * Otherwise horizontal fusion is possible if the summed threads fit a workgroup and the
      summed LDS fits a CU.
    * Does block fusion pay?  Every workgroup of a block-fused kernel is charged the LARGER side's
      static LDS and registers.  `needed` = workgroups per CU each side has resident when it runs
      alone (its grid over the CUs, capped by its own occupancy); `cap_lds` / `cap_waves` = what a
      CU holds of the fused kernel.  If both sides' needs fit a CU at once (`side_by_side`), the
      sides run in each other's shadow: fusion pays.  If not, the workgroups of the side that does
      not fit run in rounds, in whatever slots the other side leaves: with the sides' ExecTime
      known, a round of that side lasts its standalone time over its standalone rounds, and the
      fusion pays only if those rounds end within the other side's time and the side keeps at
      least half of the workgroups per CU it has alone (`bfuse_pays`).  A memory-bound side cut into short workgroups
      (LayerNorm rows, softmax rows) passes; a side whose workgroups live as long as its kernel
      (a batched GEMM resident in one round) does not: its displaced workgroups start when the
      partner ends and the pair takes as long as serial, or longer.  Without times, a side that
      does not fit is taken for short-lived only if it has neither barriers nor LDS.
    * Two sides that each keep every matrix pipe of the chip busy on their own (`matrix`: the side's inner
      loop is a stream of MFMAs; and its grid puts at least one wave on every SIMD of every CU) have
      nothing to give each other but their ends: whatever the fused form, one side's workgroups only
      take the place of the other's.  Such a pair is left unfused.  (Measured on the reference's
      benchmark arrangement -- 903 pairs of GEMMs, batched products and convolutions at batch 1024,
      all of this kind: block fusion 0.88x, thread-level fusion 0.63x, two streams 1.00x.)
    """
    ta, tb = a.dims.block[0] * a.dims.block[1] * a.dims.block[2], b.dims.block[0] * b.dims.block[1] * b.dims.block[2]
    wa, wb = -(-ta // 64), -(-tb // 64)
    hfuse_ok = not (a.HasBarriers and b.HasBarriers) and (wa + wb) * 64 <= 1024 and lds_a + lds_b <= LDS_PER_CU

    def waves_per_cu(regs):
        return 4 * min(MAX_WAVES_PER_SIMD, VGPRS_PER_SIMD // (-(-max(regs, 1) // 8) * 8))   # registers come in blocks of 8

    def wg_per_cu(waves, regs, lds):
        by_reg = waves_per_cu(regs) // max(waves, 1)
        by_lds = LDS_PER_CU // lds if lds else 1 << 30
        return max(1, min(by_reg, by_lds))

    # the fused kernel allocates max(regs) for both sides
    regs = max(a.Reg, b.Reg)
    lds = max(lds_a, lds_b)
    na, nb = wg_per_cu(wa, regs, lds), wg_per_cu(wb, regs, lds)
    ga, gb = a.dims.grid[0] * a.dims.grid[1] * a.dims.grid[2], b.dims.grid[0] * b.dims.grid[1] * b.dims.grid[2]
    rounds_a, rounds_b = -(-ga // (cus * na)), -(-gb // (cus * nb))

    # ---- does block fusion pay? -----------------------------------------------------------------
    alone = (wg_per_cu(wa, a.Reg, lds_a), wg_per_cu(wb, b.Reg, lds_b))          # occupancy of each side on its own
    per_cu = (-(-ga // cus), -(-gb // cus))
    needed = (min(alone[0], per_cu[0]), min(alone[1], per_cu[1]))
    rounds_alone = (-(-per_cu[0] // alone[0]), -(-per_cu[1] // alone[1]))
    cap_lds = LDS_PER_CU // lds if lds else 1 << 30
    cap_waves = waves_per_cu(regs)
    waves = (wa, wb)
    side_by_side = needed[0] + needed[1] <= cap_lds and needed[0] * wa + needed[1] * wb <= cap_waves
    times = (a.ExecTime, b.ExecTime)
    known = times[0] > 0 and times[1] > 0
    predicted = None
    if side_by_side:
        pays = True
        if known:
            predicted = max(times)
    else:
        # one side is dealt into the slots the other leaves; either may be that side: the better case counts
        pays = False
        for x in (0, 1):
            o = 1 - x
            slots = min(cap_lds - needed[o], (cap_waves - needed[o] * waves[o]) // waves[x])
            if known:
                life = times[x] / rounds_alone[x]                  # one round of side x's workgroups
                if slots >= 1:
                    p_x = max(times[o], -(-per_cu[x] // slots) * life)
                else:                                              # nothing of x fits beside o: x runs after it
                    p_x = times[o] + -(-per_cu[x] // max(1, min(cap_lds, cap_waves // waves[x]))) * life
                # the displaced rounds must end in the partner's shadow; if they outlast it, what is left of side
                # x runs alone at a fraction of its occupancy and the pair comes out no better than serial
                # -- and it must keep at least half of the concurrency it has alone (a side squeezed into a third
                # of its workgroups per CU, one wave at a time beside a barrier-synchronised GEMM, measured slower
                # than serial although its rounds were short)
                pays = pays or (2 * slots >= needed[x] and -(-per_cu[x] // slots) * life <= times[o])
                predicted = p_x if predicted is None else min(predicted, p_x)
            else:
                kx = (a, b)[x]
                pays = pays or (slots >= 1 and 2 * slots >= needed[x] and not kx.HasBarriers and (lds_a, lds_b)[x] == 0)
    saturates = (bool(matrix[0]) and ga * wa >= 4 * cus, bool(matrix[1]) and gb * wb >= 4 * cus)
    if saturates[0] and saturates[1]:
        pays = False
        fuse = "none"
    else:
        fuse = "hfuse" if hfuse_ok and ga == gb else ("bfuse" if pays else ("hfuse" if hfuse_ok and max(ga, gb) <= cus else "none"))
    return {"hfuse_ok": hfuse_ok, "prefer": "hfuse" if hfuse_ok and ga == gb else "bfuse",
            "wg_per_cu": (na, nb), "rounds": (rounds_a, rounds_b),
            # one chunk per round over the CUs (measured best on MI355X: the compute-bound side lands
            # one workgroup per CU and the other side is dealt on top).  A grid below the CU count
            # is then a single contiguous range, which the hardware itself deals round-robin over
            # the eight XCDs.
            "chunk": cus,
            "ratio_M": max(1, max(ga, gb) // max(1, min(ga, gb))),
            "needed": needed, "cap_lds": min(cap_lds, 1 << 20), "cap_waves": cap_waves, "side_by_side": side_by_side,
            "predicted_us": predicted, "serial_us": (times[0] + times[1]) if known else None,
            "saturates_matrix_cores": saturates,
            "bfuse_pays": pays, "fuse": fuse}
