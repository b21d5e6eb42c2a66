"""The engine against the plain implementation under every way of cutting the work.
Each case takes `env`, an object with .device, .dtype, .tol and .runner(name, pages) ->
(runner, manager, folder); the same cases run on the CPU (plain kernel twins, float32)
and on the GPU (HIP kernels, float32 and bfloat16). Every pool is filled with NaN first,
so a read of a key that the request does not own poisons its logits.
"""
from __future__ import annotations

import torch

import helpers
from helpers import Driver, plain_logits, random_ids, rel_err


def _vocab(name):
    return helpers.CONFIGS[name]["vocab_size"]


def _check(env, folder, ids, got, what):
    ref = plain_logits(folder, ids)[: got.shape[0]]
    err = rel_err(got, ref)
    assert err <= env.tol, f"{what}: error {err:.3g} > {env.tol:g}; first bad position {helpers.first_bad_row(got, ref, env.tol)}"


def whole(env, name):
    """Each request alone and whole, lengths around page and tile edges."""
    page = helpers.PAGE[name]
    for n in (1, 2, page - 1, page, page + 1, 31, 32, 33, 64, 65, 97, 130):
        runner, manager, folder = env.runner(name, -(-n // page))
        ids = random_ids(n, _vocab(name), 100 + n)
        d = Driver(runner, manager)
        d.step({"r": ids}, end=["r"])
        _check(env, folder, ids, d.result("r"), f"{name} whole n={n}")


def tail_one_by_one(env, name):
    """Most of a request in one step, its last 32 tokens one by one."""
    page = helpers.PAGE[name]
    for n in (33, 40, 100, 161):
        runner, manager, folder = env.runner(name, -(-n // page))
        ids = random_ids(n, _vocab(name), 200 + n)
        d = Driver(runner, manager)
        head = n - 32
        d.step({"r": ids[:head]})
        for t in range(head, n):
            d.step({"r": ids[t:t + 1]})
        _check(env, folder, ids, d.result("r"), f"{name} tail n={n}")


def changing_portions(env, name):
    """Portions of changing size, down to two tokens and one."""
    page = helpers.PAGE[name]
    n = 150
    ids = random_ids(n, _vocab(name), 300)
    for pattern in ([2, 3, 5, 8, 13, 21, 34, 2, 2], [17, 2, 40, 1, 1, 2, 31, 16, 16, 2], [page, page, 2, page + 1, page - 1]):
        runner, manager, folder = env.runner(name, -(-n // page))
        d = Driver(runner, manager)
        pos, i = 0, 0
        while pos < n:
            c = min(pattern[i % len(pattern)], n - pos)
            d.step({"r": ids[pos:pos + c]})
            pos += c; i += 1
        _check(env, folder, ids, d.result("r"), f"{name} portions {pattern}")


def mixed_with_reuse(env, name):
    """Up to four live requests: portions of some beside single decoded tokens of others, in a
    pool so small that pages are used again by later requests while others are still live."""
    page = helpers.PAGE[name]
    V = _vocab(name)
    lens = {"a": 70, "b": 45, "c": 33, "d": 97, "e": 58, "f": 21, "g": 80}
    ids = {r: random_ids(n, V, 400 + i) for i, (r, n) in enumerate(lens.items())}
    need = lambda r: -(-lens[r] // page)
    # pool: enough for the four largest live at once, less than all seven together
    pages = need("a") + need("d") + need("g") + need("e")
    runner, manager, folder = env.runner(name, pages)
    d = Driver(runner, manager)
    waiting = list(lens)
    live, pos = [], {}
    # chunk plan per request: a prompt part in changing portions, then the rest token by token
    portions = {"a": [30, 2, 20], "b": [45 - 12], "c": [2, 2, 9], "d": [50, 17, 2], "e": [7, 31], "f": [3], "g": [64]}
    step_i = 0
    used_again = False
    seen_pages: set = set()
    while waiting or live:
        while waiting and len(live) < 4:
            r = waiting[0]
            held = sum(len([p for p in manager.block_table(x) if p >= 0]) for x in live)
            if held + need(r) > pages:
                break
            waiting.pop(0); live.append(r); pos[r] = 0
            assert manager.allocate(r, 0, lens[r])          # reserve its pages so the plan cannot run dry
            t = set(manager.block_table(r))
            used_again |= bool(t & seen_pages)
            seen_pages |= t
        parts, ended = {}, []
        for r in live:
            plan = portions[r]
            if plan:
                c = plan.pop(0)
            else:
                c = 1
            c = min(c, lens[r] - pos[r])
            parts[r] = ids[r][pos[r]:pos[r] + c]
            pos[r] += c
            if pos[r] == lens[r]:
                ended.append(r)
        d.step(parts, end=ended)
        for r in ended:
            live.remove(r)
        step_i += 1
        assert step_i < 1000
    assert used_again, "the pool was large enough that no page was used twice: the case tests nothing"
    for r in lens:
        _check(env, folder, ids[r], d.result(r), f"{name} mixed request {r}")
    assert all(manager.num_free_pages(g) == manager.num_pages(g) for g in range(manager.num_groups))


def long_decode(env, name):
    """A short prompt, then hundreds of tokens one by one (page edges, split partitions)."""
    page = helpers.PAGE[name]
    n = 420
    ids = random_ids(n, _vocab(name), 500)
    runner, manager, folder = env.runner(name, -(-n // page))
    d = Driver(runner, manager)
    d.step({"r": ids[:3]})
    for t in range(3, n):
        d.step({"r": ids[t:t + 1]})
    _check(env, folder, ids, d.result("r"), f"{name} long decode")


def batch_of_decodes(env, name):
    """Several requests of different lengths decoding together, contexts across partition sizes."""
    page = helpers.PAGE[name]
    V = _vocab(name)
    lens = {"a": 300, "b": 17, "c": 129, "d": 64}
    ids = {r: random_ids(n + 8, V, 600 + i) for i, (r, n) in enumerate(lens.items())}
    runner, manager, folder = env.runner(name, sum(-(-(n + 8) // page) for n in lens.values()))
    d = Driver(runner, manager)
    d.step({r: ids[r][:lens[r]] for r in lens})
    for t in range(8):
        d.step({r: ids[r][lens[r] + t: lens[r] + t + 1] for r in lens})
    for r in lens:
        _check(env, folder, ids[r], d.result(r), f"{name} decode batch request {r}")


def many_rows_at_real_layer_sizes(env, name="R"):
    """Batches of 40, 12 and 3 requests at the layer sizes of a real model: their prompts in one step (a few thousand
    rows: the library's products, prefill attention at head size 128), then decode steps of as many rows (40: o and
    down in slices of K by the tiled kernel, gate/up with the gating in its epilogue; 12 and 3: the skinny products and
    their split of K, the norm inside the product), contexts in several partitions."""
    page = helpers.PAGE[name]
    V = _vocab(name)
    for count, base, steps in ((40, 90, 4), (12, 500, 4), (3, 1500, 3)):
        lens = {f"r{i}": base + 7 * i for i in range(count)}
        ids = {r: random_ids(n + steps, V, 900 + count + i) for i, (r, n) in enumerate(lens.items())}
        runner, manager, folder = env.runner(name, sum(-(-(n + steps) // page) for n in lens.values()))
        d = Driver(runner, manager)
        d.step({r: ids[r][:lens[r]] for r in lens}, want_all=False)
        for t in range(steps):
            d.step({r: ids[r][lens[r] + t: lens[r] + t + 1] for r in lens})
        for r in list(lens)[::max(1, count // 6)]:
            ref = plain_logits(folder, ids[r])[lens[r]:]
            err = rel_err(d.result(r), ref)
            assert err <= env.tol, f"{count} requests, request {r}: decode logits off by {err:.2e}"


def first_tokens(env, name):
    """The first tokens of a sequence, one by one from position 0."""
    ids = random_ids(6, _vocab(name), 700)
    runner, manager, folder = env.runner(name, 2)
    d = Driver(runner, manager)
    for t in range(6):
        d.step({"r": ids[t:t + 1]})
    _check(env, folder, ids, d.result("r"), f"{name} first tokens")


def wanted_rows_only(env, name):
    """Logits only where asked, in the order of entries and of `want`; none asked gives None."""
    from mini_engine_amd.engine.runner import StepEntry
    V = _vocab(name)
    a, b = random_ids(20, V, 800), random_ids(9, V, 801)
    runner, manager, folder = env.runner(name, 8)
    assert manager.allocate("a", 0, 20) and manager.allocate("b", 0, 9)
    out = runner.step([StepEntry("a", a, 0, [19, 0, 7]), StepEntry("b", b[:8], 0, [])])
    ref = plain_logits(folder, a)
    assert out.shape == (3, V)
    assert rel_err(out, ref[[19, 0, 7]]) <= env.tol
    out = runner.step([StepEntry("b", b[8:], 8, [0])])          # a decode entry listed alone
    assert rel_err(out, plain_logits(folder, b)[8:9]) <= env.tol
    manager.free("a")
    assert manager.allocate("a", 0, 20)
    assert runner.step([StepEntry("a", a, 0, [])]) is None


ALL = [whole, tail_one_by_one, changing_portions, mixed_with_reuse, long_decode, batch_of_decodes, first_tokens,
       wanted_rows_only]


def padded_layouts_are_used(env, name, captured: bool):
    """With `mixed_graphs_after=0` every step with a prompt portion goes through a padded layout (replayed
    from a graph where there is a GPU), single tokens alone through the decode layouts; logits as ever."""
    runner, manager, folder = env.runner(name, 40)
    assert runner.mixed_graphs is not None and runner.mixed_graphs.capture_after == 0
    V = _vocab(name)
    a, b = helpers.random_ids(70, V, 801), helpers.random_ids(45, V, 802)
    d = helpers.Driver(runner, manager)
    d.step({"a": a[:33]})
    d.step({"a": a[33:34], "b": b[:20]})
    d.step({"a": a[34:35], "b": b[20:40]})               # the same padded layout as the step before
    d.step({"a": a[35:36], "b": b[40:41]})               # two single tokens: the decode layouts
    d.step({"a": a[36:70], "b": b[41:45]})
    assert runner.mixed_graphs.replays == 4 and runner.graphs.replays == 1
    assert len(runner.mixed_graphs.captured) == 3
    if captured:
        assert all(c.graph is not None for c in runner.mixed_graphs.captured.values())
    _check(env, folder, a, d.result("a"), "a through padded layouts")
    _check(env, folder, b, d.result("b"), "b through padded layouts")


def exactly_sized_layouts_are_used(env, name, captured: bool):
    """Steps beyond the size that is padded, in which nobody decodes, keep their own token and request counts in a
    fixed layout (only the context cap and the rows of logits are rounded): a repeating pattern, portions of 40
    tokens of one prompt beside 24 of another, goes through one layout again and again while the contexts grow;
    logits as ever. `env.runner` must have made the runner with a small `mixed_graphs_max_tokens` (16) and
    `mixed_graphs_after=0`."""
    runner, manager, folder = env.runner(name, 90)
    mg = runner.mixed_graphs
    assert mg is not None and mg.capture_after == 0 and mg.max_tokens == 16 and mg.max_exact_tokens == 96
    V = _vocab(name)
    a, b, c = helpers.random_ids(130, V, 811), helpers.random_ids(201, V, 812), helpers.random_ids(130, V, 813)
    d = helpers.Driver(runner, manager)
    d.step({"c": c[:50]})                                        # 50 tokens: its own layout
    layouts = [set(mg.captured)]
    for i in range(5):                                           # 24 + 40 tokens, five times: one layout
        d.step({"a": a[24 * i:24 * i + 24], "b": b[40 * i:40 * i + 40]})
        layouts.append(set(mg.captured))
    assert len(layouts[1]) == 2 and all(l == layouts[1] for l in layouts[2:]), "the repeating step did not keep its layout"
    one = next(iter(layouts[1] - layouts[0]))
    assert (one.decode_rows, one.prefill_reqs, one.prefill_tokens) == (0, 2, 64)      # nothing was padded
    assert mg.replays == 6
    d.step({"c": c[50:51], "a": a[120:]})                        # somebody decodes beside 10 tokens: a padded layout
    d.step({"c": c[51:]})                                        # 79 tokens, nobody decodes: its own layout again
    assert mg.replays == 8 and len(mg.captured) == 4
    assert sorted(l.prefill_tokens for l in mg.captured if l.decode_rows == 0) == [50, 64, 79]
    # so many tokens with a decoding request among them get no layout of their own: the step runs as it is
    e = helpers.random_ids(41, V, 814)
    d.step({"b": b[200:], "e": e[:40]})
    assert mg.replays == 8 and len(mg.captured) == 4
    d.step({"e": e[40:]})
    if captured:
        assert all(cap.graph is not None for cap in mg.captured.values())
    _check(env, folder, a, d.result("a"), "a through exactly sized layouts")
    _check(env, folder, b, d.result("b"), "b through exactly sized layouts")
    _check(env, folder, c, d.result("c"), "c through exactly sized layouts")
    _check(env, folder, e, d.result("e"), "e beside a decoding request")
