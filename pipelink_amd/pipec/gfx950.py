"""Target profile of gfx950 (MI355X, CDNA4) in the units the resource solver works in.

Plays the part of pipec/src/pipec2/profile.py:107-186 (``SM_103A`` / ``SM_90A``): physical
capacities, which claim domains exist, how they map onto physical storage, and the launch
limits.  What differs from the NVIDIA profiles: no tensor memory and no clusters; the
"mbarrier" domain is kept under its manifest name but means 16-byte LDS slots holding
monotonically increasing 32-bit counters (there is no hardware barrier object); a "warp" is a
64-lane wavefront, so ``threads(role) = 64 * warps(role)``; registers are one unified
VGPR+AGPR file of 512 per lane at one wave per SIMD."""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass(frozen=True)
class Profile:
    name: str
    lto_arch: str
    wave_size: int
    lds_bytes: int                 # per workgroup
    max_waves_per_workgroup: int
    simds_per_cu: int
    regs_per_lane: int             # unified VGPR + AGPR at occupancy 1
    reg_granule: int
    param_limit_bytes: int         # params image a kernel may be handed
    named_barriers: int
    # claim domain -> (physical domain, bytes per unit)
    domains: dict[str, tuple[str, int]] = field(default_factory=dict)
    cta_group_legal: tuple[int, ...] = (1,)
    max_cluster: tuple[int, int, int] = (1, 1, 1)

    def physical(self, domain: str) -> tuple[str, int] | None:
        return self.domains.get(domain)

    def capacity(self, physical: str) -> int | None:
        return {"smem": self.lds_bytes, "warp": self.max_waves_per_workgroup,
                "named_barrier": self.named_barriers}.get(physical)

    def regs_cap(self, waves: int) -> int:
        """Registers per lane when `waves` wavefronts of one workgroup share a CU's SIMDs."""
        per_simd = max(1, -(-waves // self.simds_per_cu))
        return self.regs_per_lane // per_simd // self.reg_granule * self.reg_granule


GFX950 = Profile(
    name="gfx950", lto_arch="amdgcn-amd-amdhsa--gfx950", wave_size=64, lds_bytes=160 * 1024,
    max_waves_per_workgroup=16, simds_per_cu=4, regs_per_lane=512, reg_granule=8,
    param_limit_bytes=4096, named_barriers=1,
    domains={"smem": ("smem", 1), "mbarrier": ("smem", 16), "warp": ("warp", 1),
             "named_barrier": ("named_barrier", 1), "gmem_counter": ("gmem_counter", 1),
             # numbers an interpreter dispatches on; capacity comes from the pipeline (profile.py:119-126 in the reference)
             "opcode": ("opcode", 1)},
)

# The reference's own profile names are accepted when its fixtures are loaded: the checks that
# do not depend on capacities (pairing, protocol expansion, schema) behave the same.
_SM_103A = Profile(
    name="sm_103a", lto_arch="lto_103", wave_size=32, lds_bytes=232448, max_waves_per_workgroup=32,
    simds_per_cu=4, regs_per_lane=256, reg_granule=8, param_limit_bytes=32764, named_barriers=16,
    domains={"smem": ("smem", 1), "mbarrier": ("smem", 16), "warp": ("warp", 1), "tmem": ("tmem", 1),
             "named_barrier": ("named_barrier", 1), "gmem_counter": ("gmem_counter", 1)},
    cta_group_legal=(1, 2), max_cluster=(16, 16, 1),
)

PROFILES = {p.name: p for p in (GFX950, _SM_103A)}


def get_profile(name: str) -> Profile:
    from .clauses import SchemaError, reject
    if name not in PROFILES:
        reject(SchemaError, "L-ENTRYABI", "$.pipelink_abi.target.profile", f"unknown target profile {name!r}")
    return PROFILES[name]
