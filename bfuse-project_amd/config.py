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


def choose_fusion(a: KernelInfo, b: KernelInfo, lds_a: int, lds_b: int, cus: int = 256) -> dict:
    """Picks hfuse vs bfuse and a block ratio from each side's footprint.

    * Both sides with barriers -> block fusion (a wave-granular LDS barrier on both sides of
      one workgroup would have each side spin on issue slots the other needs).
    * Otherwise horizontal fusion is possible if the summed threads fit a workgroup and the
      summed LDS fits a CU.
    * The bfuse ratio interleaves in proportion to how many workgroups of each side fit a CU
      next to each other (VGPR- and LDS-limited), capped by the grid ratio.
    """
    ta, tb = a.dims.block[0] * a.dims.block[1] * a.dims.block[2], b.dims.block[0] * b.dims.block[1] * b.dims.block[2]
    wa, wb = -(-ta // 64), -(-tb // 64)
    hfuse_ok = not (a.HasBarriers and b.HasBarriers) and (wa + wb) * 64 <= 1024 and lds_a + lds_b <= LDS_PER_CU

    def wg_per_cu(waves, regs, lds):
        by_reg = (VGPRS_PER_SIMD // max(regs, 1)) * 4 // max(waves, 1)
        by_wave = MAX_WAVES_PER_SIMD * 4 // max(waves, 1)
        by_lds = LDS_PER_CU // lds if lds else 1 << 30
        return max(1, min(by_reg, by_wave, by_lds))

    # the fused kernel allocates max(regs) for both sides
    regs = max(a.Reg, b.Reg)
    na, nb = wg_per_cu(wa, regs, max(lds_a, lds_b)), wg_per_cu(wb, regs, max(lds_a, lds_b))
    ga, gb = a.dims.grid[0] * a.dims.grid[1] * a.dims.grid[2], b.dims.grid[0] * b.dims.grid[1] * b.dims.grid[2]
    rounds_a, rounds_b = -(-ga // (cus * na)), -(-gb // (cus * nb))
    return {"hfuse_ok": hfuse_ok, "prefer": "hfuse" if hfuse_ok and ga == gb else "bfuse",
            "wg_per_cu": (na, nb), "rounds": (rounds_a, rounds_b),
            # one chunk per round over the CUs (measured best on MI355X: the compute-bound side lands
            # one workgroup per CU and the other side is dealt on top).  A grid below the CU count
            # is then a single contiguous range, which the hardware itself deals round-robin over
            # the eight XCDs.
            "chunk": cus,
            "ratio_M": max(1, max(ga, gb) // max(1, min(ga, gb)))}
