"""The host side of the step function (no GPU): the integers that a step hands to the kernels, for
random mixed traces over the cache manager.  Every token's cache row must be the one its block
table names, sequences of one token come first, wanted rows follow the entries' order, and the
rows that pad a step to a fixed shape own nothing."""
import numpy as np
import pytest

import helpers
from deliverance_amd.cache.manager import CacheManager, KVGroupSpec, StateSpec
from deliverance_amd.engine.step import StepEntry, StepPacker
from deliverance_amd.sampling.sampler import RECORD_WORDS


def pack(packer, mgr, entries, pad_to=None, max_blocks=None, extra=None):
    starts = {}
    for e in entries:
        if e.rid not in mgr:
            mgr.open(e.rid)
        starts[e.rid] = mgr.extend(e.rid, len(e.tokens))
    order = sorted(range(len(entries)), key=lambda i: (len(entries[i].tokens) != 1, i))
    offs, meta, n_words = packer.layout(entries, order, pad_to=pad_to, max_blocks=max_blocks, extra=extra)
    buf = np.full(n_words, -12345, dtype=np.int32)
    packer.fill(buf, offs, meta, entries, order, starts, extra)
    assert not (buf == -12345).any(), "a word of the step was left unwritten"
    return order, starts, meta, {k: buf[a:a + n] for k, (a, n) in offs.items()}


@pytest.mark.parametrize("seed,page,groups", [(0, 16, 1), (1, 32, 2), (2, 64, 1), (3, 16, 2)])
def test_mixed_traces_pack_consistently(seed, page, groups):
    rng = np.random.default_rng(seed)
    P, V = 333, 1000
    lengths = [int(x) for x in rng.integers(1, P - 1, size=6)] + [P - 1]
    reqs = [(f"r{i}", [int(t) for t in rng.integers(0, V, size=n)]) for i, n in enumerate(lengths)]
    steps = helpers.trace_mixed(reqs, seed=seed, prefill_sizes=(9, 2, 67, 4, 130, 33), decode_tail=int(rng.integers(1, 20)))
    n_pages = helpers.max_live_tokens(steps, round_to=max(64, page)) // page
    specs = [KVGroupSpec((2 * g, 2 * g + 1), 2, 16, None) for g in range(groups)]
    mgr = CacheManager(specs, page, [n_pages] * groups, [StateSpec(9, 4)], 4)
    packer = StepPacker(mgr, groups, page)
    given = {rid: 0 for rid, _ in reqs}
    ids = dict(reqs)
    for st in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]
        if entries:
            order, starts, meta, v = pack(packer, mgr, entries)
            N, S, mb = meta["N"], meta["S"], meta["max_blocks"]
            assert N == sum(len(e.tokens) for e in entries) and S == len(entries)
            # one-token sequences first, each kind in the entries' order
            kinds = [len(entries[i].tokens) != 1 for i in order]
            assert kinds == sorted(kinds) and meta["n_decode"] == kinds.count(False)
            qs, sl = v["q_start"], v["seq_lens"]
            assert qs[0] == 0 and qs[-1] == N and (np.diff(qs) > 0).all()
            for s, i in enumerate(order):
                e = entries[i]
                rows = slice(int(qs[s]), int(qs[s + 1]))
                assert v["tokens"][rows].tolist() == list(e.tokens) == ids[e.rid][given[e.rid]:given[e.rid] + len(e.tokens)]
                assert v["positions"][rows].tolist() == list(range(given[e.rid], given[e.rid] + len(e.tokens)))
                assert (v["seq_of"][rows] == s).all() and (v["token_src"][rows] == -1).all()
                assert sl[s] == given[e.rid] + len(e.tokens)
                assert v["state_slots"][s] == mgr.state_slot(e.rid) >= 0
                for g in range(groups):
                    bt = v[f"block_table{g}"].reshape(S, mb)
                    table = mgr.table(e.rid, g)
                    assert bt[s, :len(table)].tolist() == table and (bt[s, len(table):] == -1).all()
                    assert len(table) == -(-int(sl[s]) // page) and all(0 <= p < n_pages for p in table)
                    for row, pos in zip(range(rows.start, rows.stop), v["positions"][rows]):
                        assert v[f"slot_map{g}"][row] == table[pos // page] * page + pos % page
            for g in range(groups):
                assert len(set(v[f"slot_map{g}"].tolist())) == N          # no cache row is written twice
            # wanted rows: in the order of the entries (not of the sequences) and of each entry's `want`
            first_row = {i: int(qs[s]) for s, i in enumerate(order)}
            assert v["want"].tolist() == [first_row[i] + w for i, e in enumerate(entries) for w in e.want]
            for e in entries:
                mgr.commit(e.rid)
                given[e.rid] += len(e.tokens)
        for rid in st["end"]:
            mgr.close(rid)
        mgr.check()
    assert all(pool.n_free == n_pages for pool in mgr.pools)


def test_padding_rows_own_nothing():
    """A decode step padded to a fixed shape: the added sequences have length 0, no cache row, no
    state, and their sampling records are zero."""
    page, n_pages = 16, 32
    mgr = CacheManager([KVGroupSpec((0,), 2, 16, None)], page, [n_pages])
    packer = StepPacker(mgr, 1, page)
    for rid, n in (("a", 20), ("b", 3), ("c", 40)):
        mgr.open(rid)
        mgr.extend(rid, n)
        mgr.commit(rid)
    entries = [StepEntry(rid, [7], [0]) for rid in ("a", "b", "c")]
    extra = list(range(1, 3 * RECORD_WORDS + 1))
    order, starts, meta, v = pack(packer, mgr, entries, pad_to=8, max_blocks=64, extra=extra)
    assert meta["S"] == meta["N"] == meta["R"] == 8 and meta["n_decode"] == 8 and meta["max_blocks"] == 64
    assert v["seq_lens"].tolist() == [21, 4, 41, 0, 0, 0, 0, 0]
    assert v["positions"].tolist() == [20, 3, 40, 0, 0, 0, 0, 0]
    assert (v["slot_map0"][3:] == -1).all() and (v["slot_map0"][:3] >= 0).all()
    assert (v["state_slots"] == -1).all()                 # this manager keeps no state
    assert (v["block_table0"].reshape(8, 64)[3:] == -1).all()
    assert v["want"].tolist() == list(range(8))
    assert v["extra"][:len(extra)].tolist() == extra and (v["extra"][len(extra):] == 0).all()
    assert len(v["extra"]) == 8 * RECORD_WORDS


def test_a_single_token_may_come_from_the_step_before():
    mgr = CacheManager([KVGroupSpec((0,), 1, 16, None)], 16, [8])
    packer = StepPacker(mgr, 1, 16)
    mgr.open("a"); mgr.extend("a", 5); mgr.commit("a")
    order, starts, meta, v = pack(packer, mgr, [StepEntry("a", [0], [0], from_sampled=3), StepEntry("b", [4, 5, 6], [2])])
    assert v["token_src"].tolist() == [3, -1, -1, -1] and v["positions"].tolist() == [5, 0, 1, 2]


def test_a_launch_that_fails_leaves_no_reservation_behind(tmp_path):
    """The step function reserves positions, then launches.  When the launch is refused (here: the
    kernels are asked to run on CPU tensors, which they refuse) the reservation goes back and the
    requests that the call opened are closed; a request that was open before keeps what it had."""
    import torch
    import helpers
    from deliverance_amd.engine.device_cache import DeviceCache
    from deliverance_amd.engine.step import StepEntry
    from deliverance_amd.kernels import ops
    from deliverance_amd.models.causal_lm import load_model
    from simt import harness
    m = helpers.make_model(tmp_path, helpers.CONFIG_A, 0)
    model = load_model(m.folder, torch.float32, "cpu")
    with pytest.raises(ValueError, match="page_size must be one of"):
        DeviceCache(model.cache_needs(), torch.float32, "cpu", 48, 256, n_state_slots=4)
    cache = DeviceCache(model.cache_needs(), torch.float32, "cpu", 16, 256, n_state_slots=4)
    runner = harness.make_runner(model, cache)          # the step function without pinned memory
    mgr = cache.manager
    mgr.open("old")
    mgr.extend("old", 20)
    mgr.commit("old")
    free = mgr.pools[0].n_free
    with pytest.raises((ops.KernelError, RuntimeError)):       # no GPU here: the first launch refuses
        runner.run([StepEntry("old", [1] * 30, [29]), StepEntry("new", [2] * 40, [])])
    assert mgr.live() == ["old"] and mgr.length("old") == 20 and mgr.pending("old") == 0
    assert mgr.pools[0].n_free == free
    mgr.check()
