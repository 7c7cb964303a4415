"""Pins of the CPU oracle's lattice side: Golay table, class enumeration, the
index map.  Every check here is a golden value the reference's own tests hold,
or something the mathematics fixes independently of the oracle's code."""
import numpy as np

from llvq_amd.synth import SplitMix64


def popcount(a):
    return np.array([bin(int(v)).count("1") for v in a])


# ---- Golay: llvq-core/tests/g1_invariants.rs:34-120, golay.rs:151-157 -------------
def test_generator_factorisation(orc):
    L = orc.lib()
    assert L.orc_clmul(L.orc_clmul(0xC75, 0xAE3), 0b11) == (1 << 23) | 1


def test_golay_weight_enumerator_and_order(orc):
    cw = orc.golay_codewords()
    assert len(set(cw.tolist())) == 4096
    w = popcount(cw)
    assert {k: int((w == k).sum()) for k in (0, 8, 12, 16, 24)} == {0: 1, 8: 759, 12: 2576, 16: 759, 24: 1}
    assert (w[:-1] <= w[1:]).all()  # weight-major
    for k in (8, 12, 16):
        b = cw[w == k]
        assert (b[:-1] < b[1:]).all()  # ascending inside a bucket
    assert int(cw.max()) < (1 << 24)


def test_golay_is_linear_self_dual_distance_8(orc):
    cw = orc.golay_codewords()
    s = set(cw.tolist())
    for i in range(0, 4096, 97):
        for j in range(0, 4096, 89):
            assert int(cw[i] ^ cw[j]) in s
            assert bin(int(cw[i] & cw[j])).count("1") % 2 == 0  # self-dual
    assert min(bin(int(c)).count("1") for c in cw[1:]) == 8


# ---- classes: classes.rs:284-305, leech.rs:42-54 ------------------------------------
def _tau(nmax):
    """Ramanujan tau from q prod (1 - q^n)^24."""
    c = [0] * (nmax + 1)
    c[0] = 1
    for n in range(1, nmax + 1):
        for _ in range(24):
            for k in range(nmax, n - 1, -1):
                c[k] -= c[k - n]
    return [0] + c[:nmax]  # shift by the leading q


def test_theta_series_closed_form(orc):
    """|Shell(m)| = 65520/691 (sigma_11(m) - tau(m)) for every shell of the ball."""
    L = orc.lib()
    tau = _tau(13)
    for m in range(2, 14):
        sigma11 = sum(d ** 11 for d in range(1, m + 1) if m % d == 0)
        num = 65520 * (sigma11 - tau[m])
        assert num % 691 == 0
        assert L.orc_shell_cardinality(m) == num // 691
    assert [L.orc_shell_cardinality(m) for m in (2, 3, 4, 5)] == [196560, 16773120, 398034000, 4629381120]
    assert sum(L.orc_shell_cardinality(m) for m in range(2, 14)) == orc.N13 == 280974212784720
    assert sum(L.orc_shell_cardinality(m) for m in range(2, 13)) == orc.N12 == 111043117458000


def test_class_counts(orc):
    L = orc.lib()
    infos = [orc.class_info(c) for c in range(L.orc_n_classes())]
    assert len(infos) == 383
    assert sum(1 for i in infos if i["shell"] <= 12) == 301
    assert sum(1 for i in infos if i["shell"] == 13) == 82
    assert sum(1 for i in infos if not i["odd"]) == 226 and sum(1 for i in infos if i["odd"]) == 157
    assert sum(1 for i in infos if i["shell"] == 2) == 3
    assert max(i["n_levels"] for i in infos) == 5
    # layout: contiguous, shells ascending, even before odd inside a shell
    assert infos[0]["lo"] == 1 and infos[-1]["hi"] == orc.N13
    for a, b in zip(infos, infos[1:]):
        assert b["lo"] == a["hi"] + 1
        assert (a["shell"], a["odd"]) <= (b["shell"], b["odd"])
    # shell 2 and 3 class sizes: llvq-core/tests/g1_invariants.rs:194-197, :476-566
    sizes2 = sorted(i["hi"] - i["lo"] + 1 for i in infos if i["shell"] == 2)
    assert sizes2 == sorted([97152, 1104, 98304])
    sizes3 = sorted(i["hi"] - i["lo"] + 1 for i in infos if i["shell"] == 3)
    assert sizes3 == sorted([5275648, 3108864, 98304, 8290304])
    assert L.orc_index_bits(12) == 47 and L.orc_index_bits(13) == 48


def test_flat_width_pin(orc):
    """llvq-artifact/tests/runtime_format.rs:117: the widest flat payload, 10 + 24 + 24 (L - 1)
    bits, is 130 — i.e. some class has five magnitude levels and none has six."""
    assert max(34 + 24 * (len(orc.class_levels(ci)[0]) - 1) for ci in range(383)) == 130


# ---- index map: codebook_fingerprint.rs:58, g3_index.rs, fastdec.rs tests -----------
def test_fingerprint_is_the_published_one(orc):
    assert orc.lib().orc_codebook_fingerprint() == 0x338F420F11866319


KNOWN = {
    1: [4, 4] + [0] * 22,
    196560: [-1] * 23 + [3],
    196561: [2, 2, 2, 2, 2, 4, 0, 2, 0, 0, 2, 0, -2] + [0] * 11,
    111043117458000: [-1] * 23 + [-13],
    111043117458001: [2, 2, 2, 2, 2, 4, 4, 2, 4, 4, 2, 4, -2, 4, 4, 4, 4, 4, 4, 0, 0, 0, 0, 0],
    280974212784720: [-1] * 21 + [3, 3, -13],
}


def test_known_answer_decodes(orc):
    for idx, pt in KNOWN.items():
        assert orc.index_decode(idx).tolist() == pt
        assert orc.fast_decode(idx).tolist() == pt
        assert orc.index_encode(pt) == idx


def test_origin_and_bounds(orc):
    assert orc.index_decode(0).tolist() == [0] * 24
    assert orc.index_encode([0] * 24) == 0
    assert orc.index_decode(orc.N13) is not None
    assert orc.index_decode(orc.N13 + 1) is None and orc.fast_decode(orc.N13 + 1) is None
    assert orc.index_encode([2, 2] + [0] * 22) is None  # not a lattice point
    assert orc.index_encode([16] + [0] * 23) is None  # a member beyond the ball
    assert orc.lib().orc_class_of(0) == -1 and orc.lib().orc_class_of(orc.N13 + 1) == -1
    assert orc.lib().orc_class_of(1) == 0 and orc.lib().orc_class_of(orc.N13) == 382


def test_shell2_exhaustive_and_shell3_sampled_against_enumerator(orc):
    """An enumerator that never touches the index code (llvq-core/src/shells.rs)
    lists the shell; every point must be a member, encode inside the shell's
    range without collision and come back from both decoders."""
    L = orc.lib()
    assert L.orc_shell_roundtrip_check(2, 1, 1, 196560) == 196560
    assert L.orc_shell_roundtrip_check(3, 16, 196561, 196560 + 16773120) == 16773120


def test_two_decoders_agree_on_boundaries_and_draws(orc, boundary_indices):
    a = orc.decode_many(boundary_indices, fast=True)
    b = orc.decode_many(boundary_indices, fast=False)
    assert np.array_equal(a, b)
    idx = SplitMix64(0xFA57).take(200_000) % np.uint64(orc.N13 + 1)
    assert np.array_equal(orc.decode_many(idx, fast=True), orc.decode_many(idx, fast=False))


def test_decoded_points_are_lattice_members_and_roundtrip(orc, boundary_indices):
    idx = np.concatenate([boundary_indices, SplitMix64(0x630001).take(20_000) % np.uint64(orc.N13 + 1)])
    pts = orc.decode_many(idx).astype(np.int32)
    shell = (pts.astype(np.int64) ** 2).sum(1)
    assert (shell % 16 == 0).all() and (shell // 16 <= 13).all()
    for k in range(0, idx.size, 7):
        p = pts[k]
        if int(idx[k]) != 0:
            assert orc.leech_contains(p)
        assert orc.index_encode(p) == int(idx[k])
    # the class of an index is the class whose range holds it
    for k in range(0, idx.size, 97):
        i = int(idx[k])
        if i:
            info = orc.class_info(orc.lib().orc_class_of(i))
            assert info["lo"] <= i <= info["hi"] and info["shell"] == shell[k] // 16


def test_class_levels_match_decoded_points(orc):
    for ci in range(0, 383, 3):
        info = orc.class_info(ci)
        vals, counts, nonzero = orc.class_levels(ci)
        p = np.abs(orc.index_decode((info["lo"] + info["hi"]) // 2))
        assert sorted(zip(counts, vals), reverse=True) == sorted(
            [(int((p == v).sum()), int(v)) for v in np.unique(p)], reverse=True)
        assert nonzero == int((p != 0).sum())
        assert bool(p[0] % 2) == info["odd"]
