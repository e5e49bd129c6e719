"""The figures bench.py quotes from counter runs agree with the committed rocprofv3 summaries they were read from:
a constant typed into bench.py must move when the kernel, and with it the profile, does."""
import os
import re

import helpers

PROFILES = os.path.join(helpers.ROOT, "profiles")


def _bench():
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_for_profiles", os.path.join(helpers.ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _traffic_table():
    text = open(os.path.join(PROFILES, "all_kernels_bench_configs_pmc_fetch_write.txt")).read()
    rows = {}
    for line in text.splitlines():
        m = re.match(r"^(\S.*?)\s+(\d+)\s+(\d+)\s+(\d+)\s+(\d+)\s+(\d+)\s+(\d+)\s+([\d.]+)\s+([\d.]+)$", line)
        if m:
            rows.setdefault(m.group(1).strip(), []).append(
                dict(grid=int(m.group(2)), wg=int(m.group(3)), fetch=float(m.group(8)), write=float(m.group(9))))
    return text, rows


def test_backward_kernel_traffic_constant_matches_the_counter_profile():
    """roofline.traffic of the benchmark line = FETCH_SIZE and WRITE_SIZE per dispatch of the RMSNorm backward kernel
    at the headline shape, each scaled by what the same counter reads for the 256 MiB copy kernel: recomputed here
    from the committed table, it must agree with bench.py's constant to 0.5 %."""
    text, rows = _traffic_table()
    # the headline launch: mode 1 (RMSNorm), 512-thread groups, 256 workgroups of 512 work-items
    # (last template argument false: rows on one level, the dense call)
    hits = [r for name, rs in rows.items()
            if name.startswith("norm_bwd_kernel<bf16, 1, 1, 2,") and name.endswith(", false>") for r in rs
            if r["grid"] == 256 * 512 and r["wg"] == 512]
    assert len(hits) == 1, hits
    copies = [r for name, rs in rows.items() if name.startswith("copy16_kernel") for r in rs]
    assert len(copies) == 1 and copies[0]["grid"] * 16 == 256 << 20, copies
    kib = 256 * 1024                        # what the copy kernel really moves each way
    fetch_scale = kib / copies[0]["fetch"]
    write_scale = kib / copies[0]["write"]
    assert 1.9 < fetch_scale < 2.1 and 0.99 < write_scale < 1.01          # the counters' units on this part
    traffic = (hits[0]["fetch"] * fetch_scale + hits[0]["write"] * write_scale) * 1024
    quoted = _bench().NORM_BWD_TRAFFIC_BYTES
    assert abs(quoted - traffic) <= 0.005 * traffic, (quoted, traffic)
    # and the traffic is the algorithmic bytes plus the partial rows, not a re-read: within 2 % above
    algorithmic = 32768 * (3 * 4096 * 2 + 4) + 2 * 4096 * 2
    assert 1.0 <= traffic / algorithmic < 1.02, traffic / algorithmic


def test_every_profile_names_its_command():
    """Each summary under profiles/ gives the command that made it, and that command runs committed files only."""
    for name in sorted(os.listdir(PROFILES)):
        if not name.endswith((".txt", ".md")):
            continue
        text = open(os.path.join(PROFILES, name)).read()
        cmds = [l.strip() for l in text.splitlines() if re.match(r"^\s+(rocprofv3|python3?) ", l)]
        assert cmds, name + ": no command line"
        for c in cmds:
            assert "_work" not in c and "gpurun_out" not in c, (name, c)
            for script in re.findall(r"python3?\s+(\S+\.py)", c):
                assert os.path.exists(os.path.join(helpers.ROOT, script)), (name, script)
