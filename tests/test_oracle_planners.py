"""The reference's integer planner functions (restated in oracle/planners.py) against the reference's own known
answers, and the one rule of theirs the product keeps: two workgroups per core when splitting keys."""
from oracle import planners as P


def test_shared_memory_budgets_of_the_reference_tilings():
    # test_flash.jl:84-94
    assert not P.flashfits(72, 64, 64, 256) and P.flashshared(72, 64, 64) > P.PORTABLE_SHARED_FLOOR
    assert P.flashfits(72, 64, 32, 256) and P.flashshared(72, 64, 32) <= P.PORTABLE_SHARED_FLOOR
    assert P.flashfits(72, 32, 32, 256) and P.flashfits(72, 32, 32, 128)
    # flash.jl:1170-1171: 64x32 at EP = 80 asks 48 904 bytes of the 48 KB budget, 248 to spare; 64x64 is refused
    assert P.flashcmshared(80, 64, 32) == 48904 and 48 * 1024 - 48904 == 248
    assert P.flashcmshared(80, 64, 64) > 48 * 1024
    assert P.flashcmfits(16, 32, 48 * 1024, 80, 64, 32, 256) and not P.flashcmfits(16, 32, 48 * 1024, 80, 64, 64, 256)
    assert P.flashepad(64) == 8 and P.flashepad(80) == 0


def test_crs_padding_table():
    # conv_coopmat.jl:107-110
    assert P.crsextent(147) == 160 and P.crs_admitted(147)
    assert P.crsextent(17) == 32 and not P.crs_admitted(17)
    assert P.crsextent(257) == 288 and P.crs_admitted(257)
    assert P.crsextent(769) == 800 and P.crs_admitted(769)
    assert P.crsextent(48) == 48                      # conv_coopmat.jl:50-53: 64/48 = 1.33 blows the budget, the tile pad is kept
    assert P.crsextent(588) == 608                    # config 3's patch embedding, 14 x 14 x 3


def test_key_split_rule():
    # two workgroups per core; every split a whole number of key blocks; no split when the grid already fills the device
    assert P.splitcount(48, 1, 1500, 64, 32, 20) == 4          # 20 head-rows on 48 cores: want 4, 47 blocks -> chunks of 12
    assert P.splitcount(48, 1500, 1500, 64, 32, 20) == 1
    assert P.splitcount(48, 1, 32, 64, 32, 20) == 1            # a single key block
    assert P.splitcount(0, 1, 1500, 64, 32, 20) == 1
    for (cores, Lq, Lk, BR, BC, nb) in [(256, 1, 1500, 1, 64, 20), (256, 1, 448, 1, 64, 160), (48, 23, 4096, 64, 32, 8)]:
        n = P.splitcount(cores, Lq, Lk, BR, BC, nb)
        nkb = P.cld(Lk, BC)
        chunk = P.cld(nkb, n)
        assert (n - 1) * chunk < nkb <= n * chunk             # no empty split
        assert n * P.cld(Lq, BR) * nb <= max(2 * cores, P.cld(Lq, BR) * nb) + P.cld(Lq, BR) * nb


def test_decode_attention_keeps_the_two_workgroups_per_core_rule():
    """mi_sdpa_f16_plan's split count for the rows kernel (a few query rows, or one row with a mask) aims, like
    splitcount (flash.jl:1288-1303), at two workgroups per core (256 CUs, 64-key blocks, one query row per workgroup):
    min(ceil(2 CUs / rows), blocks, 64).  Equal to the reference's count at config 5's cross-attention at batch 1;
    elsewhere never fewer splits than the reference's rule, which rounds the wanted count down and re-derives it from
    equal whole-block chunks.  A single unmasked query row takes the one-launch kernel, whose own rule is different
    (its workgroups merge inside the launch, which costs three trips to memory, so it cuts far less): at most one
    workgroup per core and a round of six 64-key passes each, nothing below nine passes."""
    import ctypes as C
    from juliavision_amd import _lib as L
    lib = L.load()

    def nsplit(E, Lq, Lk, H, B, bias=0):
        ns = C.c_int(0)
        st = L.strides4(1, E, E * Lq, E * Lq * H)
        sk = L.strides4(1, E, E * Lk, E * Lk * H)
        path = lib.mi_sdpa_f16_plan(0x10000, st, 0x20000, sk, 0x30000, sk, bias, 1, E, Lq, Lk, H, B, 0.125, C.byref(ns))
        assert L.SDPA_PATHS[path] == "rows"
        return ns.value

    assert nsplit(64, 1, 1500, 20, 1, bias=1) == P.splitcount(256, 1, 1500, 1, 64, 20) == 24
    assert nsplit(64, 1, 700, 20, 1, bias=1) == P.splitcount(256, 1, 700, 1, 64, 20) == 11
    for (Lq, Lk, H, B, bias) in [(1, 1500, 20, 4, 1), (1, 1500, 20, 8, 1), (1, 700, 20, 4, 1), (1, 1000, 20, 8, 1), (1, 4096, 8, 1, 1),
                                 (3, 100, 2, 1, 0), (23, 4096, 8, 1, 1), (5, 100, 2, 1, 0), (2, 17, 4, 1, 0), (7, 64, 1, 1, 0), (1, 100000, 1, 1, 1)]:
        rows = Lq * H * B
        mine = nsplit(64, Lq, Lk, H, B, bias)
        assert mine == max(1, min(P.cld(2 * 256, rows), P.cld(Lk, 64), 64)), (Lq, Lk, H, B)
        assert mine >= min(64, P.splitcount(256, Lq, Lk, 1, 64, H * B)), (Lq, Lk, H, B)
    # 8 to 63 unmasked queries over 512 keys or more on few (head, batch) tiles take the fused kernel on one 128-query
    # tile per (head, batch): the same two-workgroups-per-core aim, but a split is at least four 64-key blocks and there
    # are at most 32 (the reference's rule would cut the 64 blocks of its 23 x 4096 case 64 ways on 256 cores; on its own
    # 48 cores it gives 6, kernelplans.jl:300-312)
    def few(E, Lq, Lk, H, B):
        ns = C.c_int(0)
        st = L.strides4(1, E, E * Lq, E * Lq * H)
        sk = L.strides4(1, E, E * Lk, E * Lk * H)
        assert L.SDPA_PATHS[lib.mi_sdpa_f16_plan(0x10000, st, 0x20000, sk, 0x30000, sk, 0, 0, E, Lq, Lk, H, B, 0.25, C.byref(ns))] == "flash"
        return ns.value
    for (Lq, Lk, H, B) in [(23, 4096, 8, 1), (8, 512, 1, 1), (63, 100000, 4, 2), (40, 1111, 4, 2), (23, 4096, 128, 1)]:
        blocks = P.cld(Lk, 64)
        rule = max(1, min(P.cld(2 * 256, H * B), blocks // 4, 32))
        while rule > 1 and P.cld(blocks, rule) * (rule - 1) >= blocks:
            rule -= 1
        assert few(16, Lq, Lk, H, B) == rule, (Lq, Lk, H, B)
    assert few(16, 23, 4096, 8, 1) == 16 and P.splitcount(48, 23, 4096, 16, 32, 8) == 6
    # the one-launch kernel's own count
    for (Lk, H, B, want) in [(448, 20, 1, 1), (448, 20, 8, 1), (512, 20, 1, 1), (700, 20, 1, 2), (1500, 20, 1, 4), (1500, 20, 4, 3),
                             (1500, 20, 8, 1), (4096, 8, 1, 11), (100000, 1, 1, 32)]:
        passes = P.cld(Lk, 64)
        rule = 1 if passes <= 8 else max(1, min(256 // (H * B), P.cld(passes, 6), 32))
        while rule > 1 and P.cld(passes, rule) * (rule - 1) >= passes:
            rule -= 1
        assert nsplit(64, 1, Lk, H, B) == rule == want, (Lk, H, B)
