"""Integer planner functions of the reference, restated (test infrastructure, like the rest of oracle/).

They size the reference's own kernels (shared-memory budgets of its cooperative-matrix attention, K padding of
its convolution GEMM, key splits); the HIP kernels have their own tile shapes and planners, so nothing in the
product calls these.  They are here so that the tests can state which of the reference's planning rules the
product keeps (the two-workgroups-per-core split rule) and so that the reference's own known answers for them
are pinned somewhere that runs.
"""


def cld(a: int, b: int) -> int:
    return -(-a // b)


PORTABLE_SHARED_FLOOR = 48 * 1024        # flash.jl:110
GEMM_TILE = 16                           # the cooperative-matrix tile (padtile, conv_coopmat.jl:29-30)
GEMM_BK = 32                             # every staged tiling has bk = 32 (conv_coopmat.jl:32-45)


def flashshared(E: int, BQ: int, BK: int) -> int:
    """Shared bytes of the scalar fused attention (flash.jl:113)."""
    return 4 * (E * BQ + 2 * E * BK + BQ * BK + 3 * BQ)


def flashfits(E: int, BQ: int, BK: int, NT: int, sharedbudget: int = PORTABLE_SHARED_FLOOR) -> bool:
    """flash.jl:125-133."""
    if (BQ * E) % NT or (BK * E) % NT or (BQ * BK) % NT:
        return False
    if BQ > NT:
        return False
    return flashshared(E, BQ, BK) <= sharedbudget


def flashepad(EP: int) -> int:
    """flash.jl:402."""
    return 8 if EP % 32 == 0 else 0


def flashrpad(BR: int) -> int:
    """flash.jl:403."""
    return 0


def flashcmshared(EP: int, BR: int, BC: int, epad=None, rpad=None) -> int:
    """Shared bytes of the cooperative-matrix fused attention (flash.jl:339-343)."""
    epad = flashepad(EP) if epad is None else epad
    rpad = flashrpad(BR) if rpad is None else rpad
    return (2 * (EP + epad) * BR + 2 * (EP + epad) * BC + 4 * (BR + rpad) * BC + 4 * (BR + rpad) * EP
            + 2 * BC * BR + 12 * BR + 8)


def flashcmfits(tile: int, coopmatsubgroup: int, sharedbudget: int, EP: int, BR: int, BC: int, NT: int) -> bool:
    """flash.jl:411-421, with the DeviceCaps fields it reads passed one by one."""
    if BR % tile or BC % tile or EP % tile:
        return False
    if BR > NT:
        return False
    if cld((BR // tile) * (EP // tile), NT // coopmatsubgroup) > 3:
        return False
    if (BR * EP) % NT or (BC * EP) % NT or (BR * BC) % NT:
        return False
    return flashcmshared(EP, BR, BC) <= sharedbudget


def splitcount(cores: int, Lq: int, Lk: int, BR: int, BC: int, nbatch: int, allow: bool = True) -> int:
    """Key splits by llama.cpp's rule, two workgroups per core (flash.jl:1288-1303)."""
    if not allow or cores <= 0:
        return 1
    base = cld(Lq, BR) * nbatch
    if base >= 2 * cores:
        return 1
    want = max(1, (2 * cores) // base)
    if want == 1:
        return 1
    nkb = cld(Lk, BC)
    if nkb <= 1:
        return 1
    chunk = max(1, cld(nkb, want))
    n = cld(nkb, chunk)
    return 1 if n <= 1 else n


def padtile(n: int) -> int:
    return cld(n, GEMM_TILE) * GEMM_TILE


def padbk(n: int) -> int:
    return cld(n, GEMM_BK) * GEMM_BK


def crsextent(crs: int, crspad: float = 1.25) -> int:
    """The reduction extent the reference's convolution GEMM runs at (conv_coopmat.jl:60-63)."""
    p = padbk(crs)
    return p if p <= crs * crspad else padtile(crs)


def crs_admitted(crs: int, crspad: float = 1.25) -> bool:
    """crswaste veto, conv_coopmat.jl:124."""
    return crsextent(crs, crspad) <= crs * crspad
