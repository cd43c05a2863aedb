"""Hand-worked cases that pin the oracle's Bank-SR (spconv2d_utils.h:99-199) and ReorderOutChannel (:275-420).

The expected arrays below were derived by hand from the text of the reference header, step by step (the
derivations are in the comments), not by running any implementation: they hold literal lane lists and
permutations.  A dropped branch (the broadcast pass, the wait-list pads, the entry-index-as-bank comparison
of :184), a wrong tie rule or a transposed index in the cost function fails one of them.  Together with the
composition property at the end (Bank-SR on the permuted filter == both flags at once) they cover the
BANK_OPTIMIZE-only, REORDER_OUT_CHANNEL-only and combined builds.

All cases use ks = 1, so a position word is just channel << 6 (spconv2d_utils.h:91 with r = s = 0).
"""
import numpy as np
import pytest

from helpers import sparse_filter

LANES = 32


class _Product:
    """The shipped host packer (tetris_spf_create) behind the oracle's SpfPack interface, so that every hand-worked
    case below is asserted on both."""

    def __init__(self, T):
        self.T = T

    def SpfPack(self, w, tile_ic, apply_reorder, apply_vectorize, bank_optimize=False, reorder_out_channel=False):
        T = self.T
        K, C, ks, _ = w.shape
        flags = (T.BANK_OPTIMIZE if bank_optimize else 0) | (T.REORDER_OUT_CHANNEL if reorder_out_channel else 0)
        f = T.SparseFilter(w, C, K, ks, tile_ic, apply_reorder, apply_vectorize, flags)

        class R:
            offsets, stage_len, position, values, perm = f.arrays()
            bank_oob = 0
            stages = (C - 1) // tile_ic + 1

            @staticmethod
            def arrays():
                return f.arrays()
        return R


@pytest.fixture(params=["oracle", "product"])
def oracle(request):
    if request.param == "oracle":
        import oracle_py

        if not oracle_py.available():
            pytest.skip("oracle/libtetris_oracle.so not built (make -C oracle)")
        return oracle_py
    T = pytest.importorskip("tetris_amd")
    return _Product(T)


def filt(K, C, nz):
    """nz: {(k, c): value} -> OIHW filter with ks = 1"""
    w = np.zeros((K, C, 1, 1), np.float32)
    for (k, c), v in nz.items():
        w[k, c, 0, 0] = v
    return w


def emit(lane_lists, M, vec):
    """Step 2 of the constructor (:206-244) for one (group, stage): lane_lists[lane] = [(position, value), ...]."""
    L = -(-M // vec) * vec
    pos, val = [], []
    for t in range(0, L, vec):
        for lane in range(LANES):
            for it in range(vec):
                if t + it < len(lane_lists[lane]):
                    p, v = lane_lists[lane][t + it]
                else:
                    p, v = 0, 0.0
                pos.append(p)
                val.append(v)
    return L, np.array(pos, np.int32), np.array(val, np.float32)


def P(c):
    return c << 6


# ---- case A: broadcast pass, free-bank pass, wait-list pads --------------------------------------------------------
# K = 4, C = 4, TILE_IC = 4 (one stage, bank = channel).  Scan-order lists (:106-117):
#   lane0 [c0=1, c1=2]   lane1 [c0=3, c2=4]   lane2 [c1=5]   lane3 [c0=6, c1=7, c2=8]   lanes 4..31 []
# M = 3 (:118); pad budget (:121-123) = [1, 1, 2, 0] and 3 for each of the lanes 4..31.
# t=0: lane0 takes c0 (bank 0 free, :149); lane1 finds c0 already flagged this step and takes it (broadcast, :136);
#      lane2 takes c1 (bank 1); lane3 broadcast c0; lanes 4..31 have nothing -> wait list; each gets a pad on the
#      lowest free bank (:169-178): banks 0, 1 are taken, so lane o gets bank o - 2.
# t=1: lane0 takes c1 (bank 1); lane1 takes c2 (bank 2); lane2 is empty -> wait; lane3 broadcast c1;
#      wait list [2, 4..31]: lane2 pad on bank 0, lane o >= 4 on bank o - 1 (banks 0, 1, 2 taken).
# t=2: lanes 0, 1, 2 empty -> wait; lane3 takes c2 (bank 2); wait list [0, 1, 2, 4..31]: lane0 pad bank 0,
#      lane1 bank 1, lane2 bank 3 (2 is taken), lane o >= 4 bank o.
CASE_A_FILTER = filt(4, 4, {(0, 0): 1, (0, 1): 2, (1, 0): 3, (1, 2): 4, (2, 1): 5, (3, 0): 6, (3, 1): 7, (3, 2): 8})
CASE_A_LANES = [
    [(P(0), 1.0), (P(1), 2.0), (P(0), 0.0)],
    [(P(0), 3.0), (P(2), 4.0), (P(1), 0.0)],
    [(P(1), 5.0), (P(0), 0.0), (P(3), 0.0)],
    [(P(0), 6.0), (P(1), 7.0), (P(2), 8.0)],
] + [[(P(o - 2), 0.0), (P(o - 1), 0.0), (P(o), 0.0)] for o in range(4, LANES)]


@pytest.mark.parametrize("vec", [1, 4])
def test_bank_sr_broadcast_free_bank_and_pads(oracle, vec):
    p = oracle.SpfPack(CASE_A_FILTER, 4, True, vec == 4, bank_optimize=True, reorder_out_channel=False)
    L, pos, val = emit(CASE_A_LANES, 3, vec)
    assert p.bank_oob == 0
    assert p.offsets.tolist() == [0, L]
    # stage_len_ holds the lane lists' sizes after Bank-SR, pads included (:224-228), for the lanes < K only
    assert p.stage_len.tolist() == [3, 3, 3, 3] + [0] * 28
    assert p.position.tolist() == pos.tolist()
    assert p.values.tobytes() == val.tobytes()
    assert p.perm.tolist() == [0, 1, 2, 3]


# ---- case B: a lane with no pad budget left picks by the comparison of :184 as written ----------------------------
# K = 4, C = 64, TILE_IC = 64 (one stage; channels c and c + 32 share bank c).  Lists:
#   lane0 [c5=1, c6=2]   lane1 [c6=3, c7=4]   lane2 [c37=5, c38=6]   lane3 [c37=7, c38=8]     M = 2, budgets 0 0 0 0
# t=0: lane0 takes c5 (bank 5); lane1: c6 is not flagged (lane0 chose c5), bank 6 free -> c6; lane2: banks 5 and 6
#      taken, nothing flagged -> wait; lane3 likewise; lanes 4..31 wait.
#      wait list [2, 3, 4..31].  lane2 has no budget (:179): select = 0 at j = 0; at j = 1 the test is
#      bank_flag[select] > bank_flag[bank(c38)] = bank_flag[0] > bank_flag[6] = 0 > 1, false -> entry 0 = c37;
#      bank_flag[5] becomes 2.  lane3: the same walk -> c37 again (bank_flag[5] = 3).  Had :184 compared the BANK of
#      the selected entry (bank_flag[5] = 2 > bank_flag[6] = 1) lane3 would have taken c38 here: that is the quirk.
#      lanes 4..31 then get pads on the lowest free banks: 0, 1, 2, 3, 4 for lanes 4..8, then 7, 8, ... (5, 6 taken):
#      lane o >= 9 gets bank o - 2.
# t=1: lane0 takes c6 (bank 6); lane1 takes c7 (bank 7); lane2 [c38]: bank 6 taken -> wait; lane3 likewise.
#      wait list: lane2 single entry -> c38; lane3 -> c38; pads: lanes 4..9 banks 0..5, lane o >= 10 bank o - 2.
CASE_B_FILTER = filt(4, 64, {(0, 5): 1, (0, 6): 2, (1, 6): 3, (1, 7): 4, (2, 37): 5, (2, 38): 6, (3, 37): 7, (3, 38): 8})
CASE_B_LANES = [
    [(P(5), 1.0), (P(6), 2.0)],
    [(P(6), 3.0), (P(7), 4.0)],
    [(P(37), 5.0), (P(38), 6.0)],
    [(P(37), 7.0), (P(38), 8.0)],
] + [[(P(o - 4 if o <= 8 else o - 2), 0.0), (P(o - 4 if o <= 9 else o - 2), 0.0)] for o in range(4, LANES)]


def test_bank_sr_entry_index_used_as_bank(oracle):
    p = oracle.SpfPack(CASE_B_FILTER, 64, True, False, bank_optimize=True, reorder_out_channel=False)
    L, pos, val = emit(CASE_B_LANES, 2, 1)
    assert p.bank_oob == 0 and p.offsets.tolist() == [0, 2]
    assert p.position.tolist() == pos.tolist()
    assert p.values.tobytes() == val.tobytes()
    # what a "fixed" comparison would have produced for lane 3 must NOT be what we get
    assert p.position[3] == P(37) and p.position[32 + 3] == P(38)


def test_bank_sr_reorders_inside_a_lane(oracle):
    # K = 2, C = 64, TILE_IC = 64.  lane0 [c0=1, c1=2], lane1 [c32=3, c33=4].  t=0: lane0 takes c0 (bank 0); lane1: c32
    # sits on the taken bank 0, c33 on the free bank 1 -> c33 first.  t=1: lane0 c1 (bank 1), lane1 c32 (bank 0).
    # Lanes 2..31 pad on banks o and o again (t=0: banks 0, 1 taken -> lane o gets bank o; t=1 likewise).
    w = filt(2, 64, {(0, 0): 1, (0, 1): 2, (1, 32): 3, (1, 33): 4})
    p = oracle.SpfPack(w, 64, True, False, bank_optimize=True, reorder_out_channel=False)
    lanes = [[(P(0), 1.0), (P(1), 2.0)], [(P(33), 4.0), (P(32), 3.0)]] + [[(P(o), 0.0), (P(o), 0.0)] for o in range(2, LANES)]
    L, pos, val = emit(lanes, 2, 1)
    assert p.position.tolist() == pos.tolist() and p.values.tobytes() == val.tobytes()
    # without BANK_OPTIMIZE the same filter stays in scan order and lanes >= K stay empty (position 0, value 0)
    q = oracle.SpfPack(w, 64, True, False, bank_optimize=False, reorder_out_channel=False)
    plain = [[(P(0), 1.0), (P(1), 2.0)], [(P(32), 3.0), (P(33), 4.0)]] + [[] for _ in range(2, LANES)]
    L, pos, val = emit(plain, 2, 1)
    assert q.position.tolist() == pos.tolist() and q.values.tobytes() == val.tobytes()


@pytest.mark.parametrize("case", [(40, 20, 3, 8, 0.8), (64, 48, 1, 32, 0.7), (33, 70, 1, 64, 0.6), (16, 3, 7, 32, 0.85),
                                  (96, 40, 3, 16, 0.95), (70, 130, 1, 128, 0.8)])
def test_bank_sr_step_invariants(oracle, case):
    """What the text of :118-195 fixes for every (group, stage), replayed from the packed arrays: every lane emits
    exactly M items (M = longest scan-order list); a lane's zero-valued pads number M minus its non-zeros, sit on
    position b << 6 with b < 32, and no two pads of one step share a bank (each takes the lowest FREE bank); a real
    entry that shares its bank with a different position in the same step can only come from the no-budget branch
    (:179-194), i.e. all but one of the positions that meet on a bank belong to lanes whose pads were used up."""
    K, C, ks, T, sp = case
    w = sparse_filter(np.random.default_rng(K + C), K, C, ks, sp)
    p = oracle.SpfPack(w, T, True, False, bank_optimize=True, reorder_out_channel=False)
    S, G = p.stages, (K + 31) // 32
    kk = ks * ks
    for g in range(G):
        for st in range(S):
            start, M = int(p.offsets[g * S + st]), int(p.offsets[g * S + st + 1] - p.offsets[g * S + st])
            c0, c1 = st * T, min(C, (st + 1) * T)
            nnz = [int((w[g * 32 + l, c0:c1] != 0).sum()) if g * 32 + l < K else 0 for l in range(32)]
            assert M == max(nnz)
            pos = p.position[32 * start:32 * (start + M)].reshape(M, 32)
            val = p.values[32 * start:32 * (start + M)].reshape(M, 32)
            pads_before = np.zeros(32, int)
            for t in range(M):
                is_pad = val[t] == 0
                assert (pos[t][is_pad] & 63).max(initial=0) == 0 and ((pos[t][is_pad] >> 6) < 32).all()
                pad_banks = (pos[t][is_pad] >> 6).tolist()
                assert len(set(pad_banks)) == len(pad_banks)
                budget = np.array(nnz) * 0 + M - np.array(nnz) - pads_before  # pad budget of each lane at this step
                assert (budget[is_pad] > 0).all()
                by_bank = {}
                for l in range(32):
                    if not is_pad[l]:
                        by_bank.setdefault((int(pos[t][l]) >> 6) % 32, []).append((int(pos[t][l]), l))
                for items in by_bank.values():
                    distinct = sorted({q for q, _ in items})
                    if len(distinct) > 1:
                        assert any(all(budget[l] == 0 for q, l in items if q != keep) for keep in distinct), (g, st, t)
                pads_before += is_pad
            assert (pads_before == M - np.array(nnz)).all()
    assert kk >= 1


# ---- ReorderOutChannel ----------------------------------------------------------------------------------------------
def channels(spec, K, C):
    """spec: {oc: [channels with a non-zero]} -> filter (ks = 1), value = 1 + oc + c / 100"""
    return filt(K, C, {(k, c): 1.0 + k + c / 100.0 for k, cs in spec.items() for c in cs})


def perm_of(oracle, w, tile_ic):
    return oracle.SpfPack(w, tile_ic, True, True, bank_optimize=False, reorder_out_channel=True).perm.tolist()


def test_filter_gr_candidate_later_in_the_wait_list_wins_on_cost(oracle):
    # K = 24, C = 8, TILE_IC = 8: one stage, sub-groups A = [0, 8), B = [8, 16), Cc = [16, 24) (:311-324).
    #   B: oc8 has c0..c3 (count 4)            -> sub-group cost 4 (:314-321)
    #   Cc: every oc in 16..23 has c5; oc16 also c6, c7 (count 3) -> cost 3
    #   A: oc0 has c0, c1 (count 2)            -> cost 2
    # wait list order (cost descending, :303-307): B, Cc, A.  Seed B (:331-336): current_stage_mx = [4]; the positions
    # c0..c3 are flagged, current_bank_count = 1 on banks 0..3 (:345-358).
    # CalcGroupCost(Cc) (:360-391): stage_mx_nnz = 3, stage_padding = |3 - 4| = 1; c5 is new and is counted once per
    #   channel that has it -> bank 5 = 8, banks 6, 7 = 1; stage_mx_bank = 8; cost = max(8 - max(3, 4), 1) = 4.
    # CalcGroupCost(A): stage_mx_nnz = 2, stage_padding = 2; c0, c1 are flagged -> nothing new; stage_mx_bank = 1;
    #   cost = max(1 - 4, 2) = 2.   A (2) < Cc (4): A is appended although Cc comes first in the wait list; then Cc.
    w = channels({8: [0, 1, 2, 3], 16: [5, 6, 7], 17: [5], 18: [5], 19: [5], 20: [5], 21: [5], 22: [5], 23: [5], 0: [0, 1]},
                 24, 8)
    assert perm_of(oracle, w, 8) == list(range(8, 16)) + list(range(0, 8)) + list(range(16, 24))


def test_filter_gr_tie_goes_to_the_first_in_wait_list_order(oracle):
    # As above with B: oc8 has c0..c4 (count 5).  Seed B, current_stage_mx = [5].
    # Cc: cost = max(8 - max(3, 5), |3 - 5|) = max(3, 2) = 3.   A: cost = max(1 - 5, |2 - 5|) = 3.   A tie: the scan of
    # :402-410 keeps the first candidate with a strictly smaller cost, and the wait list puts Cc (sub-group cost 3)
    # before A (2) -> Cc, then A.
    w = channels({8: [0, 1, 2, 3, 4], 16: [5, 6, 7], 17: [5], 18: [5], 19: [5], 20: [5], 21: [5], 22: [5], 23: [5],
                  0: [0, 1]}, 24, 8)
    assert perm_of(oracle, w, 8) == list(range(8, 16)) + list(range(16, 24)) + list(range(0, 8))


def test_filter_gr_equal_sub_group_costs_seed_the_lower_channel(oracle):
    # K = 16, two sub-groups of equal cost 2: the wait list orders equal costs by their first channel (:306), so the
    # seed is [0, 8) and the permutation is the identity.  With cost 3 on the second sub-group it seeds instead.
    w = channels({0: [0, 1], 8: [2, 3]}, 16, 8)
    assert perm_of(oracle, w, 8) == list(range(16))
    w = channels({0: [0, 1], 8: [2, 3, 4]}, 16, 8)
    assert perm_of(oracle, w, 8) == list(range(8, 16)) + list(range(8))


def test_filter_gr_cost_sums_over_stages_with_global_channel_banks(oracle):
    # K = 24, C = 16, TILE_IC = 8: two stages; positions are built with the GLOBAL channel (:289), so stage 1's
    # channels 8..15 sit on banks 8..15.
    #   B:  oc8  stage0 c0 c1 c2 (3), stage1 c8 c9 (2)       sub-group cost 3 + 2 = 5
    #   Cc: oc16 stage0 c3 c4 c5 (3), stage1 c8 c9 (2)       cost 5 (after B in the wait list: same cost, higher channel)
    #   A:  oc0  stage0 c0 (1),       stage1 c8 c9 c10 (3)   cost 4
    # Seed B: current_stage_mx = [3, 2]; flagged c0 c1 c2 c8 c9.
    # Cc: stage0: mx 3, padding 0, new c3 c4 c5 one each, banks max 1 -> max(1 - 3, 0) = 0; stage1: mx 2, padding 0,
    #     nothing new -> max(1 - 2, 0) = 0; cost 0.
    # A:  stage0: mx 1, padding 2, nothing new -> max(1 - 3, 2) = 2; stage1: mx 3, padding 1, new c10 -> max(1 - 3, 1) = 1;
    #     cost 3.   Cc first, then A.
    w = channels({8: [0, 1, 2, 8, 9], 16: [3, 4, 5, 8, 9], 0: [0, 8, 9, 10]}, 24, 16)
    assert perm_of(oracle, w, 8) == list(range(8, 16)) + list(range(16, 24)) + list(range(0, 8))


def test_filter_gr_group_grows_past_32_when_k_is_not_a_multiple_of_8(oracle):
    # K = 36: sub-groups [0,8) [8,16) [16,24) [24,32) and the short [32,36).  oc32 has c0..c5 (count 6): highest cost,
    # seed, group size 4.  Each full sub-group has one channel with c0..c(m-1): m = 2, 5, 3, 4 for oc0, oc8, oc16, oc24.
    # Those positions are all flagged by the seed, so CalcGroupCost = max(1 - 6, |m - 6|) = 6 - m: appended in the order
    # m = 5, 4, 3 (size 4 + 24 = 28 < 32, :399) and then m = 2 as well -> one group of 36 channels.
    w = channels({32: [0, 1, 2, 3, 4, 5], 0: [0, 1], 8: [0, 1, 2, 3, 4], 16: [0, 1, 2], 24: [0, 1, 2, 3]}, 36, 8)
    assert perm_of(oracle, w, 8) == list(range(32, 36)) + list(range(8, 16)) + list(range(24, 32)) + \
        list(range(16, 24)) + list(range(0, 8))


@pytest.mark.parametrize("case", [(40, 20, 3, 8, 0.8), (64, 48, 1, 32, 0.7), (70, 70, 1, 32, 0.9), (96, 40, 3, 16, 0.95),
                                  (255, 64, 1, 128, 0.75)])
@pytest.mark.parametrize("vec", [1, 4])
def test_both_flags_equal_bank_sr_on_the_permuted_filter(oracle, case, vec):
    """The constructor applies the permutation first and Bank-SR to the permuted rows (:64-70, :110): packing with both
    flags must equal packing the row-permuted filter with BANK_OPTIMIZE alone, array for array, and the same holds for
    the plain step 1.  With the two flags pinned one at a time above, this pins their combination."""
    K, C, ks, T, sp = case
    w = sparse_filter(np.random.default_rng(K * 7 + C), K, C, ks, sp)
    perm = oracle.SpfPack(w, T, True, vec == 4, bank_optimize=False, reorder_out_channel=True).perm
    assert sorted(perm.tolist()) == list(range(K))
    for bank in (False, True):
        both = oracle.SpfPack(w, T, True, vec == 4, bank_optimize=bank, reorder_out_channel=True)
        alone = oracle.SpfPack(np.ascontiguousarray(w[perm]), T, True, vec == 4, bank_optimize=bank,
                               reorder_out_channel=False)
        assert both.perm.tolist() == perm.tolist() and alone.perm.tolist() == list(range(K))
        for a, b in zip(both.arrays()[:4], alone.arrays()[:4]):
            assert a.tobytes() == b.tobytes()
