"""The host logic of libtm_hip (tuckmill_amd/csrc/tm_hip.cpp: validation, leases,
commits, the dispatch-group planner, recorded steps, the entry point that
allocates nothing) built with g++ under the address and undefined-behaviour
sanitizers against stand-ins for the HIP runtime and for the kernels' launchers
(tests/host_cpu/), and driven through the C ABI by a small interpreter. No GPU.

What is checked is what the GPU tests cannot see directly: which launches a
sequence of operators becomes (every operator exactly once, never before
something it depends on, fused only in the forms the planner declares, fewer
launches grouped than apart), that every buffer a launch names is alive and
large enough when the launch is issued (the stand-in launchers touch them, the
sanitizer watches), the lease ledger while work is still in flight, and that
nothing is left allocated at the end. The reference's group semantics:
native/metal/tm_metal.m:654-768; the random programs are those of
tests/test_gpu_planner_random.py.
"""
import json
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HERE = os.path.join(ROOT, "tests", "host_cpu")
sys.path.insert(0, os.path.join(ROOT, "tests"))

from test_gpu_planner_random import DIMS, make_program  # noqa: E402


@pytest.fixture(scope="session")
def driver(tmp_path_factory):
    gxx = shutil.which(os.environ.get("CXX", "g++"))
    if gxx is None:
        pytest.fail("the CPU build of the host logic needs g++")
    out = str(tmp_path_factory.mktemp("host_cpu") / "driver")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-Wall", "-Wextra",
           "-Wno-format-truncation",
           "-I", HERE, "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "tuckmill_amd", "csrc"), "-o", out,
           os.path.join(ROOT, "tuckmill_amd", "csrc", "tm_hip.cpp"),
           os.path.join(HERE, "fake_runtime.cpp"), os.path.join(HERE, "stub_launch.cpp"),
           os.path.join(HERE, "driver.cpp"), "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "warning" not in res.stderr, res.stderr
    return out


def run_program(driver, lines):
    """Runs the commands; returns the parsed output lines. The sanitizers abort the
    process on a finding, the driver exits non-zero on an unexpected return code."""
    env = dict(os.environ,
               ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:halt_on_error=1:verify_asan_link_order=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    res = subprocess.run([driver], input="\n".join(lines) + "\n", capture_output=True, text=True,
                         timeout=300, env=env)
    assert res.returncode == 0, f"exit {res.returncode}\n{res.stderr[-4000:]}\n{res.stdout[-2000:]}"
    assert "Sanitizer" not in res.stderr and "runtime error" not in res.stderr, res.stderr[-4000:]
    out = [json.loads(l) for l in res.stdout.splitlines() if l.strip()]
    assert out and out[-1]["k"] == "exit"
    end = out[-1]
    # (one event per device orders the contexts' calls on the static workspace and
    # lives as long as the process)
    assert end["live_allocs"] == 0 and end["live_streams"] == 0 and end["live_graphs"] == 0 \
        and end["live_execs"] == 0 and end["live_events"] <= 1, end
    return out


def sections(out):
    """Output lines by the `mark` that precedes them."""
    cur, res = None, {}
    for o in out:
        if o["k"] == "mark":
            cur = o["text"].strip()
            res[cur] = []
        elif cur is not None:
            res[cur].append(o)
    return res


def launches_of(lines):
    return [o for o in lines if o["k"] in ("list", "single")]


# ------------------------------------------------------------ random programs --

def setup_lines(hidden, ffn, batch):
    lines = ["ctx main"]
    for kind, rows, cols in (("hh", hidden, hidden), ("hf", ffn, hidden), ("fh", hidden, ffn)):
        for i in range(2):
            lines += [f"buf {kind}{i} {rows * (cols // 32) * 34}", f"seal {kind}{i} {rows} {cols}"]
    lines.append(f"buf nw {hidden * 4}")
    for i in range(4):
        lines.append(f"buf h{i} {batch * hidden * 4}")
    for i in range(3):
        lines.append(f"buf f{i} {batch * ffn * 4}")
    lines.append("fence")
    return lines


def op_line(op, batch, hidden, ffn):
    """The driver command of one program operator, and what it reads and writes."""
    if op[0] == "product":
        _, shape, which, src, dst, call = op
        rows, cols = {"hh": (hidden, hidden), "hf": (ffn, hidden), "fh": (hidden, ffn)}[shape]
        x = ("h" if shape[0] == "h" else "f") + str(src)
        y = ("h" if shape[1] == "h" else "f") + str(dst)
        w = f"{shape}{which}"
        if call == "mma":
            cmd = f"mma {w} {x} {y} {rows} {cols} {batch} 0 0"
        elif batch == 1:
            cmd = f"gemv {w} {x} {y} {rows} {cols}"
        else:
            cmd = f"gemm {w} {x} {y} {rows} {cols} {batch} 0 0"
        return cmd, {"kind": "product", "w": w, "x": x, "y": y, "reads": {x}, "writes": {y}}
    if op[0] == "rmsnorm":
        x, y = f"h{op[1]}", f"h{op[2]}"
        return f"rmsnorm {x} nw {y} {batch} {hidden}", \
            {"kind": "rmsnorm", "x": x, "y": y, "reads": {x}, "writes": {y}}
    if op[0] in ("silu", "gelu"):
        g, u, o = f"f{op[1]}", f"f{op[2]}", f"f{op[3]}"
        return f"{op[0]} {g} {u} {o} {batch * ffn}", \
            {"kind": "glu", "g": g, "u": u, "out": o, "reads": {g, u}, "writes": {o}}
    _, width, a, y, alpha = op
    n = batch * (hidden if width == "h" else ffn)
    a, y = f"{width}{a}", f"{width}{y}"
    return f"axpy {a} {y} {alpha} {n}", \
        {"kind": "axpy", "a": a, "y": y, "reads": {a, y}, "writes": {y}}


def place_ops(ops, launches):
    """Launch index of every program operator, in program order, matching each
    operator to the first launch entry of its signature not yet taken. Fails when an
    operator has no launch or a launch entry no operator."""
    entries = []  # (launch index, signature, fused?)
    for li, l in enumerate(launches):
        if l["k"] == "single":
            bufs = l["bufs"]
            what = l["what"]
            if what == "rmsnorm":
                entries.append((li, ("rmsnorm", bufs[0], bufs[2]), False))
                if l["update"] is not None:  # h += t rides in front of the norm of h
                    entries.append((li, ("axpy", l["update"], bufs[0]), True))
            elif what in ("silu_mul", "gelu_tanh_mul"):
                entries.append((li, ("glu", bufs[0], bufs[1], bufs[2]), False))
            elif what == "f32_axpy":
                entries.append((li, ("axpy", bufs[0], bufs[1]), False))
            else:
                raise AssertionError(f"unexpected single launch {l}")
            continue
        if "norm" in l:
            entries.append((li, ("rmsnorm", l["norm"]["x"], l["norm"]["y"]), True))
        for i, p in enumerate(l["ops"]):
            entries.append((li, ("product", p["w"], p["x"], p["y"]), False))
            if "residual" in p:
                entries.append((li, ("axpy", p["y"], p["residual"]), True))
            if "glu" in p:
                entries.append((li, ("glu", p["y"], l["ops"][i + 1]["y"], p["glu"]), True))
    taken = [False] * len(entries)
    placed = []
    for op in ops:
        if op["kind"] == "product":
            sig = ("product", op["w"], op["x"], op["y"])
        elif op["kind"] == "rmsnorm":
            sig = ("rmsnorm", op["x"], op["y"])
        elif op["kind"] == "glu":
            sig = ("glu", op["g"], op["u"], op["out"])
        else:
            sig = ("axpy", op["a"], op["y"])
        for k, (li, esig, fused) in enumerate(entries):
            if not taken[k] and esig == sig:
                taken[k] = True
                placed.append((li, fused))
                break
        else:
            raise AssertionError(f"operator {sig} has no launch; launches: {launches}")
    assert all(taken), [e for e, t in zip(entries, taken) if not t]
    return placed


def check_order(ops, placed):
    """No operator runs before one it depends on; two dependent operators share a
    launch only as a declared fusion (the later one rides in the earlier one's
    launch, or the earlier one is the norm fused in front)."""
    for j, b in enumerate(ops):
        for i in range(j):
            a = ops[i]
            depends = (a["writes"] & (b["reads"] | b["writes"])) or (a["reads"] & b["writes"])
            if not depends:
                continue
            (la, fa), (lb, fb) = placed[i], placed[j]
            assert la <= lb, (i, j, a, b, placed)
            if la == lb:
                assert fa or fb, f"dependent operators {a} and {b} share launch {la} unfused"


RATIOS = []


@pytest.mark.parametrize("dims", DIMS, ids=lambda d: f"{d[0]}x{d[1]}")
@pytest.mark.parametrize("with_mma", [False, True], ids=["exact", "mma"])
def test_random_programs_become_the_same_operators_in_a_valid_order(driver, dims, with_mma):
    hidden, ffn = dims
    n_programs = 24 if with_mma else 32
    for seed in range(n_programs):
        rng = np.random.default_rng((2000 if with_mma else 1000) + seed)
        if with_mma:
            batch = int(rng.choice([17, 40, 64, 100, 128, 256, 512]))
        else:
            batch = int(rng.choice([1, 1, 2, 3, 4, 8, 20, 32]))
        program = make_program(rng, batch, with_mma)
        cmds, ops = zip(*(op_line(op, batch, hidden, ffn) for op in program))
        lines = setup_lines(hidden, ffn, batch)
        lines += ["mark apart", *cmds, "fence", "stats"]
        lines += ["mark group", "begin", *cmds, "end", "fence", "stats"]
        lines += ["mark recorded", "begin", *cmds, "record s"]
        lines += ["mark replay", "run s", "run s", "fence", "stepfree s", "stats"]
        sec = sections(run_program(driver, lines))
        apart, group, recorded = (launches_of(sec[k]) for k in ("apart", "group", "recorded"))
        # apart: one launch per operator, in order
        placed = place_ops(ops, apart)
        assert [p[0] for p in placed] == list(range(len(ops))) and not any(p[1] for p in placed)
        # grouped: every operator once, dependencies respected, fewer launches
        check_order(ops, place_ops(ops, group))
        assert len(group) <= len(apart)
        RATIOS.append((len(group), len(apart)))
        # recorded: the same plan, every launch inside the recording, no stop events
        strip = lambda ls: [{k: v for k, v in l.items() if k != "recording"} for l in ls]
        assert strip(recorded) == strip(group)
        assert all(l["recording"] for l in recorded) and not any(l["recording"] for l in group)
        for name in ("apart", "group", "replay"):
            stats = [o for o in sec[name] if o["k"] == "stats"][-1]
            assert stats["in_flight"] == 0 and stats["committed"] == stats["completed"], (name, stats)
        replay = [o for o in sec["replay"] if o["k"] == "stats"][-1]
        assert replay["graph_launches"] == 2 and replay["live_graphs"] == 0 and replay["live_execs"] == 0


def test_zz_grouped_programs_took_far_fewer_launches():
    assert RATIOS
    assert sum(g for g, _ in RATIOS) < 0.8 * sum(a for _, a in RATIOS), RATIOS


# ------------------------------------------------------------------ lifetimes --

W = 1024 * 32 * 34  # a 1024 x 1024 Q8_0 matrix


def test_buffers_freed_inside_an_open_group_live_until_the_commit_completes(driver):
    lines = ["ctx main", f"buf w {W}", "seal w 1024 1024", "buf x 4096", "buf y 4096", "buf h 4096",
             "fence", "mark base", "stats",
             "begin", "gemv w x y 1024 1024", "axpy y h 1.0 1024", "free x", "free y", "free w",
             "free h",
             "mark open", "stats", "end", "mark committed", "stats",
             "advance 1000", "mark advanced", "stats", "fence", "mark fenced", "stats"]
    sec = sections(run_program(driver, lines))
    st = {k: [o for o in v if o["k"] == "stats"][0] for k, v in sec.items()}
    assert st["base"]["allocated"] == W + 3 * 4096 and st["base"]["in_flight"] == 0
    # the handles are gone, the group still holds the memory
    assert st["open"]["allocated"] == 0 and st["open"]["live_allocs"] == st["base"]["live_allocs"]
    # ... then the commit does, visibly, until its stop event is reached
    assert st["committed"]["in_flight"] == W + 3 * 4096
    assert st["committed"]["live_allocs"] == st["base"]["live_allocs"]
    assert st["advanced"]["in_flight"] == 0 and st["advanced"]["completed"] == st["advanced"]["committed"]
    assert st["advanced"]["live_allocs"] == st["base"]["live_allocs"] - 4
    assert st["fenced"]["in_flight"] == 0
    launch = launches_of(sec["open"] + sec["committed"])
    assert len(launch) == 1 and launch[0]["ops"][0]["residual"] == "h"  # the update rode along


def test_abort_and_destroy_release_what_an_open_group_holds(driver):
    lines = ["ctx main", f"buf w {W}", "buf x 4096", "buf y 4096", "fence", "mark base", "stats",
             "begin", "gemv w x y 1024 1024", "free w", "free x", "mark held", "stats",
             "abort", "mark aborted", "stats", "!abort", "!end",
             # a second group is left open when the context goes
             f"buf w2 {W}", "buf x2 4096", "begin", "gemv w2 x2 y 1024 1024", "free w2",
             "!fence", "!upload y 0 16", "destroy main", "mark destroyed", "stats"]
    sec = sections(run_program(driver, lines))
    st = {k: [o for o in v if o["k"] == "stats"][0] for k, v in sec.items()}
    assert st["held"]["live_allocs"] == st["base"]["live_allocs"]
    assert st["aborted"]["live_allocs"] == st["base"]["live_allocs"] - 2
    assert not launches_of(sec["held"] + sec["aborted"])  # nothing was ever issued
    assert st["destroyed"]["live_allocs"] == 0 and st["destroyed"]["live_streams"] == 0


def test_a_recorded_step_keeps_its_buffers_and_goes_with_its_context(driver):
    lines = ["ctx main", f"buf w {W}", "seal w 1024 1024", "buf x 4096", "buf y 4096", "buf h 4096",
             "buf nw 4096", "fence", "mark base", "stats",
             "begin", "rmsnorm h nw x 1 1024", "gemv w x y 1024 1024", "axpy y h 1.0 1024",
             "record s", "free w", "free x", "free y", "mark recorded", "stats",
             "run s", "run s", "advance 1000", "mark ran", "stats",
             "!record t",                      # no group is open
             "begin", "!run s", "abort",       # not inside a group
             # a second step is never freed: the context disposes of it
             f"buf w2 {W}", "begin", "gemv w2 h nw 1024 1024", "record t", "free w2",
             "destroy main", "mark destroyed", "stats"]
    sec = sections(run_program(driver, lines))
    st = {k: [o for o in v if o["k"] == "stats"][0] for k, v in sec.items()}
    assert st["recorded"]["allocated"] == 8192  # h and nw
    assert st["recorded"]["live_allocs"] == st["base"]["live_allocs"]  # the step holds the rest
    assert st["ran"]["graph_launches"] == 2 and st["ran"]["in_flight"] == 0
    rec = launches_of(sec["base"] + sec["recorded"])
    # the norm rides in front of the product that reads it; the update of h does not ride
    # behind it, because the launch itself still reads h for that norm
    assert len(rec) == 2 and all(l["recording"] for l in rec)
    assert rec[0]["norm"] == {"x": "h", "y": "x"} and rec[0]["ops"][0]["normed"]
    assert "residual" not in rec[0]["ops"][0] and rec[1]["what"] == "f32_axpy"
    assert st["destroyed"]["live_allocs"] == 0 and st["destroyed"]["live_execs"] == 0


def test_the_entry_point_that_allocates_nothing_allocates_nothing(driver):
    rows, cols, batch = 6144, 2048, 512
    wbytes = rows * (cols // 32) * 34
    lines = ["ctx a", f"buf w {wbytes}", f"seal w {rows} {cols}", f"buf x {batch * cols * 4}",
             f"buf y {batch * rows * 4}", "fence", "mark base", "stats",
             f"mma_noalloc w x y {rows} {cols} {batch} 0 0", "mark called", "stats",
             "begin", f"!mma_noalloc w x y {rows} {cols} {batch} 0 0", "abort",
             f"!mma_noalloc w x y 4096 8192 512 0 0",  # sealed as 6144 x 2048
             # a second context on the same device: ordered behind the first one's call
             "ctx b", f"buf wb {wbytes}", f"seal wb {rows} {cols}", f"buf xb {batch * cols * 4}",
             f"buf yb {batch * rows * 4}", "fence", "mark base_b", "stats",
             f"mma_noalloc wb xb yb {rows} {cols} {batch} 0 0", "use a",
             f"mma_noalloc w x y {rows} {cols} {batch} 0 0", "use b", "fence", "use a", "fence",
             "mark done", "stats"]
    sec = sections(run_program(driver, lines))
    st = {k: [o for o in v if o["k"] == "stats"][0] for k, v in sec.items()}
    assert st["called"]["live_allocs"] == st["base"]["live_allocs"], "a device allocation was made"
    assert st["called"]["committed"] == st["base"]["committed"], "the call is not a commit"
    assert st["called"]["in_flight"] == wbytes + batch * (cols + rows) * 4
    call = [o for o in sec["base"] + sec["called"] if o["k"] in ("list", "zero_words")]
    assert [o["k"] for o in call] == ["zero_words", "list"] and call[1]["variant"] == "bf16x3"
    assert call[1]["ops"][0]["chunks"] > 1  # partial tiles and counters from the static workspace
    assert st["done"]["in_flight"] == 0


def test_allocation_failures_leave_the_context_usable_and_leak_nothing(driver):
    rows, cols, batch = 6144, 2048, 512
    wbytes = rows * (cols // 32) * 34
    lines = ["ctx main", f"buf w {wbytes}", f"seal w {rows} {cols}", f"buf x {batch * cols * 4}",
             f"buf y {batch * rows * 4}", "fence", "mark base", "stats",
             "failmalloc 1", "buf ok 64", "!buf never 64", "failmalloc 0",
             # the bf16 product's workspace cannot grow: the commit fails, nothing is issued
             "failmalloc 1", "buf spare 64", "mark fail", f"!mma w x y {rows} {cols} {batch} 0 0",
             "failmalloc 0", "fence", "stats",
             "mark work", f"mma w x y {rows} {cols} {batch} 0 0", "fence", "stats"]
    sec = sections(run_program(driver, lines))
    st = {k: [o for o in v if o["k"] == "stats"][0] for k, v in sec.items()}
    assert not launches_of(sec["fail"])
    assert st["fail"]["in_flight"] == 0 and st["fail"]["committed"] == st["fail"]["completed"]
    assert st["fail"]["live_allocs"] == st["base"]["live_allocs"] + 2  # ok and spare
    work = launches_of(sec["work"])
    assert len(work) == 1 and work[0]["variant"] == "bf16x3"
    assert st["work"]["in_flight"] == 0
    assert st["work"]["live_allocs"] > st["fail"]["live_allocs"]  # the workspace it could now grow


# ------------------------------------------------------- volume and the rest --

def test_long_queues_of_commits_retire_and_are_measured(driver):
    """Commits that pile up while nothing completes: every one borrows its
    predecessor's stop event as its start, more than a thousand retire at one fence
    (their events are read in batches), and the measurement entry points see them."""
    n = 1500
    per_commit = W + 8192  # a commit leases every allocation it names
    lines = ["ctx main", f"buf w {W}", "seal w 1024 1024", "buf x 4096", "buf y 4096", "fence",
             "profile 1", "commitlog 1", "stats", "mark run"]
    lines += ["gemv w x y 1024 1024"] * n
    lines += ["stats", "mark some", "advance 800", "stats", "download_after y 0 64 300",
              f"!download_after y 0 64 {n + 100}", "mark fenced", "fence", "stats", "measure",
              "profile 0", "commitlog 0"]
    out = run_program(driver, lines)
    base = [o for o in out if o["k"] == "stats"][0]
    sec = sections(out)
    st = {k: [o for o in v if o["k"] == "stats"][0] for k, v in sec.items()}
    assert st["run"]["committed"] - base["committed"] == n
    assert st["run"]["completed"] == base["completed"] and st["run"]["in_flight"] == n * per_commit
    done = st["some"]["completed"] - base["completed"]
    assert 0 < done < n and st["some"]["in_flight"] == (n - done) * per_commit
    assert st["fenced"]["completed"] == st["fenced"]["committed"] and st["fenced"]["in_flight"] == 0
    measured = [o for o in out if o["k"] == "measure"][0]
    assert measured["logged"] == n and measured["profile_count"] == n
    assert measured["profile_slots"] == 1  # "q8_0_gemv:1024x1024"
    # the events went back to the pool: two per commit at most were ever alive
    assert st["fenced"]["live_events"] <= n + 8


def test_a_decode_step_of_many_products_and_a_prefill_layer_as_groups(driver):
    """197 independent GEMVs in one launch, 300 in two (the list holds 224); a prefill
    layer whose products alternate between kernels keeps one open launch per kernel
    while nothing depends on anything; batches of 17-32 tokens over a column tail go
    as two descriptors per product; F16 and int8 products and the small operators
    mix into a group without sharing launches they cannot share."""
    lines = ["ctx main", f"buf w {W}", "seal w 1024 1024"]
    for i in range(300):
        lines += [f"buf x{i} 4096", f"buf y{i} 4096"]
    lines += ["fence", "mark step197", "begin"]
    lines += [f"gemv w x{i} y{i} 1024 1024" for i in range(197)]
    lines += ["end", "fence", "mark step300", "begin"]
    lines += [f"gemv w x{i} y{i} 1024 1024" for i in range(300)]
    lines += ["end", "fence", "mark tail", "stats"]
    # Gemma widths at 24 tokens through the exact product: two token groups each
    gw = 1152 * (6912 // 32) * 34
    lines += [f"buf gw {gw}", "seal gw 1152 6912", f"buf gx {24 * 6912 * 4}", f"buf gy {24 * 1152 * 4}",
              "mark groups24", f"gemm gw gx gy 1152 6912 24 0 0", "fence", "mark setup"]
    # a layer at 512 tokens: q,k,v and gate,up (bf16 kernels) around o and down
    M, hid, ffn = 512, 1024, 3072
    for name, r, c in (("q", 2048, hid), ("k", 1024, hid), ("v", 1024, hid), ("o", hid, 2048),
                       ("gate", ffn, hid), ("up", ffn, hid), ("down", hid, ffn)):
        lines += [f"buf W{name} {r * (c // 32) * 34}", f"seal W{name} {r} {c}",
                  f"buf X{name} {M * c * 4}", f"buf Y{name} {M * r * 4}"]
    lines += ["mark layer", "begin"]
    lines += [f"mma W{n} X{n} Y{n} {r} {c} {M} 0 0" for n, r, c in
              (("q", 2048, hid), ("k", 1024, hid), ("v", 1024, hid), ("o", hid, 2048),
               ("gate", ffn, hid), ("up", ffn, hid), ("down", hid, ffn))]
    lines += ["end", "fence", "stats", "mark setup2"]
    # other families in one group
    lines += [f"buf f16w {256 * 100 * 2}", f"buf fx {4 * 100 * 4}", f"buf fy {4 * 256 * 4}",
              f"buf xq {8 * 1024 + 32 * 8 * 4}", f"buf iy {8 * 1024 * 4}", "buf part 512", "buf tok 16",
              "buf ck 8192", "buf rowout 4096",
              "mark families", "begin", "f16gemm f16w fx fy 256 100 4 0 0",
              "quant Xq xq 1024 8 0", "i8 w xq iy 1024 1024 8 0", "i8fma w xq iy 1024 1024 8 0",
              "argmax iy 8192 part tok 1", "checksum w 0 1024 ck", "row w rowout 5 1024 0",
              "scale rowout rowout 0.5 1024", "end", "fence", "stats"]
    sec = sections(run_program(driver, lines))
    one = launches_of(sec["step197"])
    assert len(one) == 1 and len(one[0]["ops"]) == 197 and one[0]["variant"] == "decode"
    two = launches_of(sec["step300"])
    assert [len(l["ops"]) for l in two] == [224, 76]
    g24 = launches_of(sec["groups24"])
    assert len(g24) == 1 and g24[0]["variant"] == "split" and g24[0]["p"][1] == 4  # 4 tokens a wave
    layer = launches_of(sec["layer"])
    assert len(layer) == 1 and layer[0]["variant"] == "bf16x3" and layer[0]["p"][0] == 2
    assert [p["chunks"] for p in layer[0]["ops"]] == [1, 1, 1, 2, 1, 1, 3]
    fam = launches_of(sec["families"])
    kinds = [(l["k"], l.get("variant") or l["what"]) for l in fam]
    assert kinds == [("list", "f16"), ("single", "q8_0_quantize_act"), ("list", "i8_lds"),
                     ("list", "i8_lds"), ("single", "argmax_f32"), ("single", "xor_checksum_u32"),
                     ("single", "q8_0_row"), ("single", "f32_scale")], kinds
    assert fam[2]["p"][1] == 0 and fam[3]["p"][1] == 1  # the fused tail never shares a launch
    for name in ("tail", "layer", "families"):
        stats = [o for o in sec[name] if o["k"] == "stats"][-1]
        assert stats["in_flight"] == 0


def test_the_no_allocation_calls_are_refused_past_their_lease_list(driver):
    rows, cols, batch = 3072, 1024, 8  # a vector-kernel product: no workspace, still leased
    wbytes = rows * (cols // 32) * 34
    lines = ["ctx main", f"buf w {wbytes}", f"seal w {rows} {cols}", f"buf x {batch * cols * 4}",
             f"buf y {batch * rows * 4}", "fence", "mark calls"]
    lines += [f"mma_noalloc w x y {rows} {cols} {batch} 0 0"] * 1024
    lines += ["stats", f"!mma_noalloc w x y {rows} {cols} {batch} 0 0", "fence", "mark again",
              f"mma_noalloc w x y {rows} {cols} {batch} 0 0", "copy y 0 x 0 16", "stats", "fence", "stats"]
    sec = sections(run_program(driver, lines))
    stats = [o for o in sec["calls"] if o["k"] == "stats"][0]
    per_call = wbytes + batch * (cols + rows) * 4
    assert stats["in_flight"] == 1024 * per_call
    after = [o for o in sec["again"] if o["k"] == "stats"]
    # the commit behind the call adopts its leases (and adds its own on x and y)
    assert after[0]["in_flight"] == per_call + batch * (cols + rows) * 4 and after[1]["in_flight"] == 0


def test_a_ragged_last_round_is_cut_off_as_a_tail_segment(driver):
    """300 whole-K units on the 256 workgroup slots of the 128-token tile (76800 x
    1024 at 128 tokens) are a full round and one that is a sixth full: the units of
    the last round become a tail segment of rows whose K is cut in chunks
    (q8::bx3_plan_launch). A launch with many rounds (the 151936 x 1024 vocabulary
    at 512 tokens: 2376 units; at 128 tokens: 594, where the estimate gains too
    little) keeps its K whole everywhere, and so does the 64-token tile, where
    tails do not pay. The recording launcher checks the segment against the limits."""
    rows, cols = 151936, 1024
    lines = ["ctx main", f"buf w {rows * (cols // 32) * 34}", f"seal w {rows} {cols}",
             f"buf w2 {76800 * (cols // 32) * 34}", f"seal w2 76800 {cols}",
             f"buf x {512 * cols * 4}", f"buf y {512 * rows * 4}", "fence",
             "mark t128", f"mma w2 x y 76800 {cols} 128 0 0", "fence",
             "mark noalloc", f"mma_noalloc w2 x y 76800 {cols} 128 0 0", "fence",
             "mark m64", f"mma w x y {rows} {cols} 64 0 0", "fence",
             "mark m128", f"mma w x y {rows} {cols} 128 0 0", "fence",
             "mark m512", f"mma w x y {rows} {cols} 512 0 0", "fence", "stats"]
    lines += ["mark m32", f"mma w x y {rows} {cols} 32 0 0", "fence", "mark m17", f"mma w x y {rows} {cols} 17 0 0",
              "fence"]
    sec = sections(run_program(driver, lines))
    for name in ("m32", "m17"):  # up to 32 tokens: the 32-token tiles behind the same split pass
        (l,) = launches_of(sec[name])
        assert l["variant"] == "bf16x3" and l["p"][0] == 1 and l["small_tiles"] is True, l
    for name in ("t128", "noalloc"):
        (l,) = launches_of(sec[name])
        assert l["variant"] == "bf16x3" and l["p"][0] == 2, l
        tail = l["tail"]
        assert tail["product"] == 0 and tail["row_tiles"] == 44 and 2 <= tail["chunks"] <= 3, l
        assert l["ops"][0]["chunks"] == 1
    for name in ("m64", "m128", "m512"):
        (l,) = launches_of(sec[name])
        assert "tail" not in l and l["ops"][0]["chunks"] == 1
        assert l["small_tiles"] is False  # (33 tokens and more: the staged kernel itself)


def test_small_prefill_launches_behind_their_operator_take_its_split_form(driver):
    """A layer at 128 tokens as an executor encodes it: every product launch has too
    few work units for the staged bf16 kernel. The launches right behind the norm or
    the gated activation that writes their one input (q,k,v; gate,up; down) run the
    f32 kernel's tiles on the bf16 matrix cores, fed with the split form that the
    operator leaves (fuse_split_passes); o, whose input no operator of the group
    writes, stays on the f32 kernel, and so does everything over raw weights or when
    the operator's result is read from an offset."""
    M, hid, ffn = 128, 1024, 3072
    lines = ["ctx main", f"buf nw {hid * 4}", f"buf h {M * hid * 4}", f"buf xn {(M * hid + 32) * 4}",
             f"buf act {M * ffn * 4}"]
    mats = (("q", 2048, hid), ("k", 1024, hid), ("v", 1024, hid), ("o", hid, 2048),
            ("gate", ffn, hid), ("up", ffn, hid), ("down", hid, ffn))
    for name, r, c in mats:
        lines += [f"buf W{name} {r * (c // 32) * 34}", f"seal W{name} {r} {c}", f"buf Y{name} {M * r * 4}",
                  f"buf R{name} {r * (c // 32) * 34}"]

    def layer(prefix, x_off=0):
        return ["begin", f"rmsnorm h nw xn {M} {hid}",
                f"mma {prefix}q xn Yq 2048 {hid} {M} {x_off} 0", f"mma {prefix}k xn Yk 1024 {hid} {M} {x_off} 0",
                f"mma {prefix}v xn Yv 1024 {hid} {M} {x_off} 0",
                f"mma {prefix}o Yq Yo {hid} 2048 {M} 0 0", f"axpy Yo h 1.0 {M * hid}",  # (o reads q: no attention here)
                f"rmsnorm h nw xn {M} {hid}",
                f"mma {prefix}gate xn Ygate {ffn} {hid} {M} {x_off} 0",
                f"mma {prefix}up xn Yup {ffn} {hid} {M} {x_off} 0",
                f"silu Ygate Yup act {M * ffn}", f"mma {prefix}down act Ydown {hid} {ffn} {M} 0 0",
                f"axpy Ydown h 1.0 {M * hid}", "end", "fence"]

    lines += ["fence", "mark sealed"] + layer("W") + ["mark raw"] + layer("R") + ["mark offset"] + \
             layer("W", x_off=32) + ["mark recorded", "begin"] + layer("W")[1:-2] + ["record s", "run s", "fence",
                                                                                   "stepfree s", "stats"]
    sec = sections(run_program(driver, lines))

    def shape(ls):
        return [(l["k"], l.get("variant") or l["what"], l.get("split", False)) for l in ls]

    # (the gated activation rides in the launch of gate and up, which leaves its split
    # form for the down projection behind its own input's: 7 launches)
    want = [("single", "rmsnorm", True), ("list", "mma_split", False), ("list", "mma_f32", False),
            ("single", "rmsnorm", True), ("list", "mma_split", False), ("list", "mma_split", False),
            ("single", "f32_axpy", False)]
    got = launches_of(sec["sealed"])
    assert shape(got) == want, shape(got)
    assert [len(l["ops"]) for l in got if l["k"] == "list"] == [3, 1, 2, 1]
    assert all(l["presplit"] == 1 for l in got if l.get("variant") == "mma_split")
    pair, down = got[4], got[5]
    assert "glu" in pair["ops"][0] and pair["split_out"] and pair["xs_in_off"] == 0
    assert down["xs_in_off"] == M * hid * 6 and "glu" not in down["ops"][0]
    assert shape([l for l in launches_of(sec["recorded"]) if l.get("recording")]) == want
    for name in ("raw", "offset"):
        ls = launches_of(sec[name])
        # (with the norm's result read from an offset, the down projection still takes the
        # gated activation's whole result)
        last = "mma_f32" if name == "raw" else "mma_split"
        assert [l["variant"] for l in ls if l["k"] == "list"] == ["mma_f32"] * 3 + [last], shape(ls)
        splits = [l.get("split", False) for l in ls if l["k"] == "single"]
        assert splits == ([False] * 4 if name == "raw" else [False, False, True, False]), shape(ls)


def test_a_staged_gated_pair_up_to_256_tokens_takes_the_fused_small_tiles(driver):
    """Gate and up of the 0.6B layer at 256 tokens have enough work for the staged bf16
    kernel's 64-token tile when they stand alone. Behind their norm and in front of the
    gated activation and a down projection that stays on the small tiles, the pair takes
    the small tiles too, with the activation in its launch (three launches where four
    stood); at 512 tokens (the large tile, a staged down projection) nothing changes."""
    hid, ffn = 1024, 3072
    lines = ["ctx main", f"buf nw {hid * 4}", f"buf h {512 * hid * 4}", f"buf xn {512 * hid * 4}",
             f"buf act {512 * ffn * 4}", f"buf Yg {512 * ffn * 4}", f"buf Yu {512 * ffn * 4}",
             f"buf Yd {512 * hid * 4}"]
    for name, r, c in (("gate", ffn, hid), ("up", ffn, hid), ("down", hid, ffn)):
        lines += [f"buf W{name} {r * (c // 32) * 34}", f"seal W{name} {r} {c}"]

    def half(M):
        return ["begin", f"rmsnorm h nw xn {M} {hid}", f"mma Wgate xn Yg {ffn} {hid} {M} 0 0",
                f"mma Wup xn Yu {ffn} {hid} {M} 0 0", f"silu Yg Yu act {M * ffn}",
                f"mma Wdown act Yd {hid} {ffn} {M} 0 0", "end", "fence"]

    lines += ["fence", "mark alone", "begin", f"mma Wgate xn Yg {ffn} {hid} 256 0 0",
              f"mma Wup xn Yu {ffn} {hid} 256 0 0", "end", "fence",
              "mark m256"] + half(256) + ["mark m512"] + half(512) + ["stats"]
    sec = sections(run_program(driver, lines))
    (alone,) = launches_of(sec["alone"])
    assert alone["variant"] == "bf16x3" and alone["p"][0] == 1
    m256 = launches_of(sec["m256"])
    assert [(l["k"], l.get("variant") or l["what"]) for l in m256] == \
        [("single", "rmsnorm"), ("list", "mma_split"), ("list", "mma_split")], m256
    assert "glu" in m256[1]["ops"][0] and m256[1]["split_out"] and m256[2]["xs_in_off"] == 256 * hid * 6
    m512 = launches_of(sec["m512"])
    assert [(l["k"], l.get("variant") or l["what"]) for l in m512] == \
        [("single", "rmsnorm"), ("list", "bf16x3"), ("single", "silu_mul"), ("list", "bf16x3")], m512


def test_few_token_products_that_are_large_together_leave_the_vector_kernel(driver):
    """Products of 13 M weights each at 16 tokens through the MFMA entry point: alone a
    product stays on the token-split vector kernel (too small for the 32-token tiles to
    pay), four of them in one group (50 M weights) go to the bf16 path's small tiles behind
    one split pass. The same products through the exact entry point, or with a residual
    update riding in the launch, stay where they are."""
    rows, cols, M = 6144, 2048, 16
    lines = ["ctx main", f"buf x {M * cols * 4}", f"buf h {M * rows * 4}"]
    for i in range(4):
        lines += [f"buf w{i} {rows * (cols // 32) * 34}", f"seal w{i} {rows} {cols}", f"buf y{i} {M * rows * 4}"]
    lines += ["fence", "mark alone", f"mma w0 x y0 {rows} {cols} {M} 0 0", "fence",
              "mark group", "begin"] + [f"mma w{i} x y{i} {rows} {cols} {M} 0 0" for i in range(4)] + ["end", "fence",
              "mark exact", "begin"] + [f"gemm w{i} x y{i} {rows} {cols} {M} 0 0" for i in range(4)] + ["end", "fence",
              "mark fused", "begin"] + [f"mma w{i} x y{i} {rows} {cols} {M} 0 0" for i in range(4)] + \
             [f"axpy y3 h 1.0 {M * rows}", "end", "fence", "stats"]
    sec = sections(run_program(driver, lines))
    (alone,) = launches_of(sec["alone"])
    assert alone["variant"] == "split"
    (group,) = launches_of(sec["group"])
    assert group["variant"] == "bf16x3" and group["p"][0] == 1 and group["small_tiles"] is True
    assert len(group["ops"]) == 4 and group["presplit"] == 0
    (exact,) = launches_of(sec["exact"])
    assert exact["variant"] == "split"
    fused = launches_of(sec["fused"])
    assert fused[0]["variant"] == "split" and "residual" in fused[0]["ops"][3], fused


# ------------------------------------------------------------------ threads --

def test_two_contexts_and_their_readers_on_four_threads_under_the_thread_sanitizer(tmp_path):
    """What the library promises about threads (tests/host_cpu/threads.cpp): two
    owner threads drive a context each (groups, calls that allocate nothing on the
    one static workspace, frees with work in flight, fences) while a reader thread
    per context calls tm_hip_download_after and the dispatch counters, which take
    no lock in the reference's typed layer (crates/metal/src/lib.rs:2618-2633)."""
    gxx = shutil.which(os.environ.get("CXX", "g++"))
    out = str(tmp_path / "threads")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-fno-omit-frame-pointer", "-Wall",
           "-Wextra", "-Wno-format-truncation", "-I", HERE, "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "tuckmill_amd", "csrc"), "-o", out,
           os.path.join(ROOT, "tuckmill_amd", "csrc", "tm_hip.cpp"),
           os.path.join(HERE, "fake_runtime.cpp"), os.path.join(HERE, "stub_launch.cpp"),
           os.path.join(HERE, "threads.cpp"), "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:exitcode=66")
    run = subprocess.run([out, "300"], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, f"exit {run.returncode}\n{run.stderr[-6000:]}"
    assert "ThreadSanitizer" not in run.stderr, run.stderr[-6000:]
    end = json.loads(run.stdout.strip().splitlines()[-1])
    assert end["k"] == "exit" and end["failures"] == 0 and end["enqueued"] > 1000
