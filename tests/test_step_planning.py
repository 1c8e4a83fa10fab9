"""The step's arrays, planned for all entries at once, against the same arrays made entry by entry and row by row from
their definitions: which token, position, block-table line and cache slot every row of every stage gets, which row of
the previous stage a lagging stage's row reads, and where the wanted places lie."""
import random

import numpy as np
import pytest
import torch

from tiny_inference_server_amd.cache import CacheManager
from tiny_inference_server_amd.engine.batch import Entry, plan_step_batch
from tiny_inference_server_amd.parts.spec import PagedKvNeed


def arrays_of(plan):
    pk = plan.packer
    get = lambda i: pk.parts[i].reshape(pk.offsets[i][1])
    out = []
    for pl in plan.plans:
        out.append({k: (get(pl[k]) if pl[k] is not None else None) for k in ("tokens", "positions", "row_seq", "cu", "source", "keep_src", "keep_slot", "want")}
                   | {"ws": {g: get(i) for g, i in pl["ws"].items()}, "valid": pl["valid"], "seq_rows": pl["seq_rows"],
                      "max_kv": pl["max_kv"], "max_rows": pl["max_rows"], "n_rows": pl["n_rows"],
                      "keep_count": pl["keep_count"], "previous_rows": pl["previous_rows"]})
    return {g: get(i) for g, i in plan.bt_ids.items()}, get(plan.slots_id), out


def row_by_row(entries, lags, has_source, cache):
    """The definitions, one row at a time."""
    ps = cache.page_size
    stages, prev = [], None
    for j, lag in enumerate(lags):
        rows = []                                          # (entry, position, token)
        first_of, seq_rows = {}, []
        for k, e in enumerate(entries):
            first_of[k] = len(rows)
            mine = [(k, p, e.tokens[p + lag - e.start]) for p in range(max(0, e.start - lag), e.start + len(e.tokens) - lag)]
            rows += mine
            seq_rows.append((first_of[k], max(0, e.start - lag), len(mine)))
        st = dict(tokens=[t for _, _, t in rows], positions=[p for _, p, _ in rows], row_seq=[k for k, _, _ in rows],
                  seq_rows=seq_rows, n_rows=len(rows))
        st["ws"] = {g: [grp.tables[entries[k].slot][p // ps] * ps + p % ps for k, p, _ in rows] for g, grp in cache.groups.items()}
        if has_source[j]:
            where = {(k, p): r for r, (k, p, _) in enumerate(prev)}
            st["source"] = [where.get((k, p), -(entries[k].slot + 1)) for k, p, _ in rows]
            last = {}
            for r, (k, p, _) in enumerate(prev):
                last[k] = r
            st["keep_src"] = [last[k] for k in sorted(last)]
            st["keep_slot"] = [entries[k].slot for k in sorted(last)]
        want, valid = [], []
        for k, e in enumerate(entries):
            for i in e.want:
                p = e.start + i - lag
                r = [r for r, (kk, pp, _) in enumerate(rows) if kk == k and pp == p]
                want.append(r[0] if r else -1)
                valid.append(bool(r))
        st["want"], st["valid"] = want, valid
        stages.append(st)
        prev = rows
    return stages


@pytest.mark.parametrize("seed", range(12))
def test_arrays_for_all_entries_at_once_equal_the_definitions(seed):
    rng = random.Random(seed)
    ps = rng.choice([2, 4, 16])
    window = rng.choice([0, 0, 7])
    needs = {"a": PagedKvNeed(2, 8), "b": PagedKvNeed(1, 16, window=window)}
    cache = CacheManager(needs, ps, 400, 12, torch.float32, "cpu", allocate=False)
    lags, has_source = [0, 1, 2][:rng.choice([1, 2, 3])], [False, True, True]
    entries = []
    for _ in range(rng.randint(1, 9)):
        slot = cache.open_request()
        start = rng.choice([0, 0, 1, 2, 3, 17, 40])
        n = rng.choice([1, 1, 1, 2, 3, 9, 33])
        cache.grow(slot, start + n)
        if window:
            cache.release_behind(slot, start, max_lag=2)          # pages behind the window are gone (-1 in the table)
        toks = [rng.randrange(1000) for _ in range(n)]
        want = sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))
        entries.append(Entry(slot, start, toks, want))
    rng.shuffle(entries)
    width = rng.choice([None, 64])
    plan = plan_step_batch(entries, lags, has_source[:len(lags)], cache, 4096, None, table_width=width)
    tables, slots, got = arrays_of(plan)
    assert slots.tolist() == [e.slot for e in entries]
    for g, grp in cache.groups.items():
        for k, e in enumerate(entries):
            line = grp.tables[e.slot]
            assert tables[g][k, :len(line)].tolist() == [max(p, 0) for p in line] and not tables[g][k, len(line):].any()
        assert width is None or tables[g].shape[1] == width
    want = row_by_row(entries, lags, has_source, cache)
    for j, (a, b) in enumerate(zip(got, want)):
        for key in ("tokens", "positions", "row_seq", "want"):
            assert a[key].tolist() == b[key], (j, key)
        assert a["valid"] == b["valid"] and a["seq_rows"] == b["seq_rows"] and a["n_rows"] == b["n_rows"]
        assert a["cu"].tolist() == [0] + [f + n for f, _, n in b["seq_rows"]]
        for g in cache.groups:
            # a row behind a window group's released pages would write to a page that is gone: such rows do not come
            # (new positions are never behind the window), so compare where the page is still held
            held = [v >= 0 for v in b["ws"][g]]
            assert [x for x, h in zip(a["ws"][g].tolist(), held) if h] == [x for x, h in zip(b["ws"][g], held) if h]
        if has_source[j]:
            assert a["source"].tolist() == b["source"] and a["keep_src"].tolist() == b["keep_src"]
            assert a["keep_slot"].tolist() == b["keep_slot"] and a["keep_count"] == len(b["keep_src"])
            assert a["previous_rows"] == sum(s >= 0 for s in b["source"])
        live = [(p0 + n, n) for _, p0, n in b["seq_rows"] if n > 0]
        assert a["max_kv"] == max([x for x, _ in live] or [0]) and a["max_rows"] == max([n for _, _, n in b["seq_rows"]] or [0])


def test_a_step_beyond_the_context_is_refused_before_anything_is_planned():
    cache = CacheManager({"a": PagedKvNeed(1, 8)}, 4, 50, 2, torch.float32, "cpu", allocate=False)
    s = cache.open_request()
    cache.grow(s, 40)
    with pytest.raises(ValueError, match="beyond the model's context of 32"):
        plan_step_batch([Entry(s, 30, [1, 2, 3], [2])], [0], [False], cache, 32, None)
    with pytest.raises(ValueError, match="want index 3"):
        plan_step_batch([Entry(s, 3, [1, 2, 3], [3])], [0], [False], cache, 64, None)
