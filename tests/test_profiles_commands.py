"""The commands quoted in profiles/*.md must run committed files only: every `bench.py --only LEG` names a leg that
bench.py implements, every script path exists in the tree, and the profile summaries bench.py cites exist."""
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def bench_legs():
    src = (ROOT / "bench.py").read_text()
    legs = set(re.findall(r'args\.only == "([a-z0-9-]+)"', src))
    for group in re.findall(r"args\.only in \(([^)]*)\)", src):
        legs.update(re.findall(r'"([a-z0-9-]+)"', group))
    return legs


def test_profile_commands_name_existing_legs_and_files():
    legs = bench_legs()
    assert {"sweep", "sweep-b4", "moe", "moe-t", "copy", "single"} <= legs
    seen = 0
    for md in sorted((ROOT / "profiles").glob("*.md")):
        for line in md.read_text().splitlines():
            if "rocprofv3" not in line or " -- " not in line:
                continue
            seen += 1
            program = line.split(" -- ", 1)[1].split()
            assert program[0] in ("python3", "python"), (md.name, line)
            assert (ROOT / program[1]).is_file(), (md.name, program[1])
            if "--only" in program:
                assert program[program.index("--only") + 1] in legs, (md.name, line)
    assert seen >= 20


def test_traffic_sources_cited_by_bench_exist():
    src = (ROOT / "bench.py").read_text()
    cited = set(re.findall(r'"(profiles/[A-Za-z0-9_./-]+\.md)"', src))
    assert cited
    for path in cited:
        assert (ROOT / path).is_file(), path


def test_every_only_leg_is_listed_in_the_help_text():
    src = (ROOT / "bench.py").read_text()
    help_line = re.search(r'"--only".*help="([^"]+)"', src).group(1)
    listed = set(re.findall(r"[a-z0-9]+(?:-[a-z0-9]+)*", help_line.split(":", 1)[1]))
    assert bench_legs() <= listed, bench_legs() - listed
