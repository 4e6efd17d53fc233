"""The host library (csrc/host.cpp) on the CPU: the step's integer buffer against a
layout computed here independently, the preparation of decode steps, the uniform
streams."""


import numpy as np
import pytest
import torch

from zig_ai_amd.cache import FREED, CacheManager
from zig_ai_amd.engine import StepEntry, StepError, build_step
from zig_ai_amd.kernels import host as hostlib
from zig_ai_amd.parts import PagedNeed, StateNeed
from zig_ai_amd.sampling import UniformStream, uniforms

CPU = torch.device("cpu")


def manager(num_pages=40, page_size=4, num_slots=4, window=0):
    needs = {0: StateNeed((8, 3)), 1: PagedNeed.kv(2, 16, 0), 3: PagedNeed.kv(2, 16, 0)}
    if window:
        needs[4] = PagedNeed.kv(2, 16, window)
    return CacheManager(needs, page_size, num_pages, num_slots, allocate=False)


def expected_layout(m, entries, grans, min_pages=0):
    """What the buffer must hold, from the cache manager's own answers."""
    out = {"token_ids": [], "positions": [], "token_seq": [], "seq_start": [0], "ctx_len": [],
           "slot_id": [], "logit_rows": []}
    width = max([len(m.table(e.request, g.index)) for e in entries for g in m.groups] + [1, min_pages])
    for g in m.groups:
        out[f"slots{g.index}"] = []
        out[f"table{g.index}"] = []
    for gran in grans:
        out[f"iseq{gran}"], out[f"irow{gran}"], out[f"icnt{gran}"] = [], [], []
    row = 0
    for s, e in enumerate(entries):
        ctx, n = m.num_tokens(e.request), len(e.tokens)
        out["token_ids"] += list(e.tokens)
        out["positions"] += list(range(ctx, ctx + n))
        out["token_seq"] += [s] * n
        out["ctx_len"].append(ctx)
        out["slot_id"].append(m.slot_of(e.request))
        out["logit_rows"] += [row + w for w in e.want]
        for g in m.groups:
            table = m.table(e.request, g.index)
            out[f"slots{g.index}"] += [table[p // m.page_size] * m.page_size + p % m.page_size
                                       for p in range(ctx, ctx + n)]
            out[f"table{g.index}"] += table + [FREED] * (width - len(table))
        for gran in grans:
            for done in range(0, n, gran):
                out[f"iseq{gran}"].append(s)
                out[f"irow{gran}"].append(row + done)
                out[f"icnt{gran}"].append(min(gran, n - done))
        row += n
        out["seq_start"].append(row)
    return out, width


@pytest.mark.parametrize("window", [0, 6])
def test_step_buffer_matches_an_independent_layout(window):
    m = manager(window=window)
    for r in ("a", "b", "c"):
        m.admit(r)
    # request a already holds 13 tokens (pages behind the window were given back)
    m.reserve("a", 13)
    m.commit("a", 13)
    m.reserve("b", 5)
    m.commit("b", 5)
    entries = [StepEntry("b", [7, 8, 9, 10, 11, 12, 13], [6]), StepEntry("a", [3], [0]),
               StepEntry("c", [1, 2], [0, 1])]
    for e in entries:
        m.reserve(e.request, len(e.tokens))
    grans = (2, 5)
    ctx = build_step(entries, m, CPU, 100, grans, min_pages=3)
    want, width = expected_layout(m, entries, sorted(grans), min_pages=3)
    assert ctx.table_width == width and ctx.n_tokens == 10 and ctx.n_seqs == 3
    assert ctx.n_logit_rows == 4 and ctx.max_keys == 14
    for name, values in want.items():
        off, n = ctx.offsets[name]
        assert off % 4 == 0, name
        assert ctx.host[off:off + n].tolist() == values, name
    if window:
        assert FREED in m.table("a", 1)          # the windowed group gave pages back
    assert ctx.block_tables[0].shape == (3, width)
    seq, row0, cnt, n_items = ctx.items[5]
    assert n_items == 4 and cnt.tolist() == [5, 2, 1, 2]
    # the same entries give the same layout whatever the cache holds: sections only
    again = build_step(entries, m, CPU, 100, grans, min_pages=3)
    assert again.offsets == ctx.offsets and np.array_equal(again.host, ctx.host)


def test_step_errors_name_the_request():
    m = manager()
    m.admit("a")
    m.reserve("a", 4)
    with pytest.raises(StepError, match="'a'.*vocabulary"):
        build_step([StepEntry("a", [100], [0])], m, CPU, 100)
    with pytest.raises(StepError, match="'a'.*place 2"):
        build_step([StepEntry("a", [1, 2], [2])], m, CPU, 100)
    with pytest.raises(StepError, match="not admitted"):
        build_step([StepEntry("zz", [1], [0])], m, CPU, 100)
    with pytest.raises(StepError, match="twice"):
        build_step([StepEntry("a", [1], [0]), StepEntry("a", [1], [0])], m, CPU, 100)
    with pytest.raises(StepError, match="no tokens"):
        build_step([StepEntry("a", [], [])], m, CPU, 100)
    with pytest.raises(StepError, match="not reserved"):
        build_step([StepEntry("a", [1] * 5, [])], m, CPU, 100)
    with pytest.raises(StepError, match="max_position"):
        build_step([StepEntry("a", [1, 2, 3], [])], m, CPU, 100, max_position=2)
    with pytest.raises(StepError, match="at least one"):
        build_step([], m, CPU, 100)
    m.check()


def test_decode_preparation_takes_pages_for_all_or_none():
    m = manager(num_pages=3, page_size=4)
    lib = hostlib.lib()
    for r, n in (("a", 4), ("b", 3)):
        m.admit(r)
        m.reserve(r, n)
        m.commit(r, n)
    m.admit("c")
    m.reserve("c", 4)
    m.commit("c", 4)                      # all three pages are taken now
    reqs = np.array([m.handles.of(r) for r in ("b", "a")], dtype=np.int64)
    toks = np.array([5, 6], dtype=np.int32)
    extent = np.zeros((2,), dtype=np.int64)
    rc = lib.za_decode_prepare(m.native, 2, reqs.ctypes.data, toks.ctypes.data, 100, 0,
                               extent.ctypes.data)
    assert rc == hostlib.OUT_OF_PAGES      # a needs a second page, none is free
    assert len(m.table("a", 0)) == 1 and len(m.table("b", 0)) == 1
    m.release("c")
    rc = lib.za_decode_prepare(m.native, 2, reqs.ctypes.data, toks.ctypes.data, 100, 0,
                               extent.ctypes.data)
    assert rc == 0 and extent.tolist() == [2, 5]
    assert len(m.table("a", 0)) == 2 and len(m.table("b", 0)) == 1
    toks[1] = 100
    assert lib.za_decode_prepare(m.native, 2, reqs.ctypes.data, toks.ctypes.data, 100, 0,
                                 extent.ctypes.data) == hostlib.STEP
    assert "vocabulary" in hostlib.last_error()
    m.check()


def test_uniform_streams():
    a = uniforms([42] * 4096, [3] * 4096, range(4096))
    assert a == uniforms([42] * 4096, [3] * 4096, range(4096))           # a pure function
    assert all(0.0 <= u < 1.0 for u in a)
    assert UniformStream(42, 3).at(17) == a[17]
    x = np.asarray(a)
    assert abs(x.mean() - 0.5) < 0.02 and abs(x.std() - 12 ** -0.5) < 0.01
    assert len(set(a)) > 4000
    # another seed, another request: other numbers, uncorrelated with the first
    for other in (uniforms([43] * 4096, [3] * 4096, range(4096)),
                  uniforms([42] * 4096, [4] * 4096, range(4096))):
        y = np.asarray(other)
        assert abs(np.corrcoef(x, y)[0, 1]) < 0.06
    # consecutive numbers of one stream are uncorrelated too
    assert abs(np.corrcoef(x[:-1], x[1:])[0, 1]) < 0.06
    # large keys are taken whole
    assert uniforms([2 ** 63 + 5], [2 ** 40], [2 ** 33]) != uniforms([5], [2 ** 40], [2 ** 33])


def test_context_split_plan():
    """How decode attention cuts long contexts: a function of the batch shape and the
    longest context only; ranges cover the context, are multiples of the key tile,
    and there are never more than SPLIT_MAX of them."""
    from zig_ai_amd.parts.attention import SPLIT_MAX, SPLIT_TARGET, plan_split
    for items in (1, 2, 8, 33, 64, 200):
        for kv_heads in (1, 8):
            for max_keys in (1, 100, 513, 2048, 4096, 33000, 131072, 1 << 20):
                keys, nsplit = plan_split(items, kv_heads, max_keys)
                assert (keys, nsplit) == plan_split(items, kv_heads, max_keys)
                if nsplit == 1:
                    assert keys == 0
                    continue
                assert keys % 64 == 0
                assert keys * nsplit >= max_keys > keys * (nsplit - 1)
                assert nsplit <= SPLIT_MAX
    assert plan_split(64, 8, 100000) == (0, 1)            # enough requests: no cut
    assert plan_split(8, 8, 2200) == (576, 4)             # the benchmark's decode step
    keys, nsplit = plan_split(1, 8, 131072)               # one long request: ~SPLIT_TARGET groups
    assert (keys, nsplit) == (4096, 32) and 8 * nsplit >= SPLIT_TARGET
    assert plan_split(16, 8, 4608) == (2304, 2)           # ranges of the same length
    assert plan_split(12, 8, 3072) == (1536, 2)           # never more workgroups than SPLIT_TARGET
    assert plan_split(20, 8, 8192) == (0, 1) and plan_split(7, 8, 3072)[1] == 4
    assert plan_split(1, 8, 1024) == (256, 4)             # short contexts are cut finer
    assert plan_split(1, 8, 3072) == (512, 6) and plan_split(1, 8, 512) == (0, 1)
