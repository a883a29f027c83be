"""The global-load addresses of the GEMM kernel that takes tiles past the edge of C,
restated on the CPU (ulmblas_amd/csrc/gemm_kernel.hip.h: `Stage`, the 32-bit
packet offsets of SHARED kernels, the packet moved back along x, the tail
slab): every element a thread reads must lie inside the operand's window
[0, (cols-1)*ld + rows), for every thread, packet and tile, in all four
transpositions, for shapes whose last tile holds one row or column, fewer
than a packet, or nearly a whole tile.  (A kernel that reads past an operand
faults the GPU; this is the check that runs before it gets there.)"""
import itertools

import pytest


def stage(X, BK, NT, KCONTIG, VEC):
    L = X*BK//NT//VEC; XV = X//VEC; XC_SMALL = (NT % XV == 0); KV = BK//VEC; KROWS = NT//16; KC_SMALL = (KROWS % KV == 0)
    def x0(t):
        if not KCONTIG: return VEC*(t % XV if XC_SMALL else t)
        return (t%16) + 16*((t//16)//KV) if KC_SMALL else (t%16)
    def k0(t):
        if not KCONTIG: return t//XV if XC_SMALL else 0
        return VEC*((t//16)%KV if KC_SMALL else (t//16))
    def dx(i):
        if not KCONTIG: return 0 if XC_SMALL else VEC*NT*(i % (XV//NT))
        return 16*(KROWS//KV)*i if KC_SMALL else 16*(i//(KV//KROWS))
    def dk(i):
        if not KCONTIG: return (NT//XV)*i if XC_SMALL else i//(XV//NT)
        return 0 if KC_SMALL else VEC*KROWS*(i % (KV//KROWS))
    return L, x0, k0, dx, dk

def check_operand(name, X, BK, NT, KCONTIG, VEC, extent_x, K, ld, esize):
    """operand with x extent `extent_x` (m or n), k extent K; stored with stride (sx, sk)."""
    L, x0, k0, dx, dk = stage(X, BK, NT, KCONTIG, VEC)
    sx, sk = (ld, 1) if KCONTIG else (1, ld)
    size = (extent_x - 1)*sx + (K - 1)*sk + 1      # elements of the window, last one included
    XBIAS = 0 if KCONTIG else VEC - 1
    tiles = (extent_x + X - 1)//X
    nwhole = K//BK
    bad = 0
    for tile in range(tiles):
        x00 = tile*X
        x_last = min(X, extent_x - x00) - 1
        for t in range(NT):
            for i in range(L):
                if KCONTIG: x = min(x0(t)+dx(i), x_last)
                else: x = min(x0(t), x_last + 1 - VEC)
                off = ((x + XBIAS)*sx + (k0(t)+dk(i))*sk)*esize
                assert 0 <= off < 2**32, (name, "offset range", off)
                for slab in ([0, nwhole-1] if nwhole > 0 else []):
                    base = x00*sx + slab*BK*sk - XBIAS*sx           # element index of origin (biased)
                    first = base + off//esize
                    for e in range(VEC):
                        idx = first + e
                        if not (0 <= idx < size):
                            bad += 1
                            if bad < 5: print("OOB", name, dict(tile=tile, t=t, i=i, slab=slab, e=e, idx=idx, size=size, x=x, x_last=x_last))
                # the tail slab
                if K % BK:
                    slab = nwhole
                    for e in range(VEC):
                        kk = k0(t)+dk(i)+(e if KCONTIG else 0)
                        if slab*BK + kk < K:
                            idx = x00*sx + slab*BK*sk - XBIAS*sx + off//esize + e
                            if not (0 <= idx < size):
                                bad += 1
                                if bad < 5: print("OOB tail", name, tile, t, i, e, idx, size)
    return bad



CONFIGS = [("d256x128", 256, 128, 16, 512, 2, 8), ("d128x128", 128, 128, 16, 256, 2, 8),
           ("s256x256", 256, 256, 16, 512, 4, 4), ("s256x128", 256, 128, 16, 256, 4, 4)]
SHAPES = [(257, 129, 17), (130, 4, 33), (6, 5, 40), (4, 4, 16), (515, 131, 20), (259, 258, 16)]


@pytest.mark.parametrize("config", CONFIGS, ids=lambda c: c[0])
def test_every_packet_stays_inside_its_operand(config):
    nm, BM, BN, BK, NT, VEC, es = config
    bad = 0
    for (m, n, k) in SHAPES:
        for ta, tb in itertools.product((0, 1), repeat=2):
            for pad in (0, 3):
                lda = (k if ta else m) + pad
                ldb = (n if tb else k) + pad
                bad += check_operand(f"{nm} A ta={ta} {m}x{n}x{k}", BM, BK, NT, bool(ta), VEC, m, k, lda, es)
                bad += check_operand(f"{nm} B tb={tb} {m}x{n}x{k}", BN, BK, NT, not tb, VEC, n, k, ldb, es)
    assert bad == 0


def test_the_check_sees_an_unbiased_offset():
    """Without the bias of VEC-1 places a packet moved back from the first
    place of a tile gets a negative offset, which the kernel would use as an
    unsigned one: the model must notice."""
    L, x0, k0, dx, dk = stage(256, 16, 512, False, 2)
    x_last = 0                                   # a tile with a single valid row
    x = min(x0(0), x_last + 1 - 2)
    assert x == -1 and (x + 1) >= 0
