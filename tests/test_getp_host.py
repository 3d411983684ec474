"""Host side of the batch runtime without a device: the request file, the output file and the
exact-match verifier of host/moe_getp.hpp against the formats of the reference's
src/getp/eval.cpp (:42-100, :109-206), through the built program host/bin/moe_stack_main."""
import os
import subprocess

import pytest

from conftest import ROOT

EXE = os.path.join(ROOT, "gpt-oss-amd_amd", "host", "bin", "moe_stack_main")

# shaped like the reference's tests/references/input.txt: a count, then one prompt per line
PROMPTS = ["What is the biggest misconception about tidal power?",
           "Explain tidal power to a 5-year-old.",
           "",
           "List the top 5 challenges in tidal power today.",
           "Write a 150-word explainer on tidal power & its grid: costs, \"quotes\", tabs\tand all."]


def run(*args):
    if not os.path.exists(EXE):
        pytest.fail("%s is missing: run __graft_entry__.build()" % EXE)
    return subprocess.run([EXE] + [str(a) for a in args], capture_output=True, text=True)


def write_requests(path, prompts, count=None):
    with open(path, "w") as f:
        f.write("%d\n" % (len(prompts) if count is None else count))
        for p in prompts:
            f.write(p + "\n")


def expected_tokens(prompts, max_seq_len):
    out = []
    for i, p in enumerate(prompts):
        n = min(len(p) % 7 + 1, max_seq_len)
        out.append([len(p)] + [i + j - 1 for j in range(1, n)])
    return out


def test_request_file_round_trip(tmp_path):
    write_requests(tmp_path / "in.txt", PROMPTS)
    r = run("requests", tmp_path / "in.txt", tmp_path / "out.txt", 32)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "num requests: 5" in r.stdout
    lines = open(tmp_path / "out.txt").read().split("\n")
    assert lines[-1] == "" and len(lines) == 6          # one line per request, each newline-terminated
    want = expected_tokens(PROMPTS, 32)
    assert [[int(t) for t in l.split(" ")] for l in lines[:-1]] == want
    assert all("  " not in l and not l.endswith(" ") for l in lines)   # single spaces, none trailing


def test_request_file_truncation_short_files_and_long_lines(tmp_path):
    write_requests(tmp_path / "in.txt", PROMPTS)
    r = run("requests", tmp_path / "in.txt", tmp_path / "out.txt", 32, 2)      # truncate_lines = 2
    assert r.returncode == 0 and "num requests: 2" in r.stdout
    assert len(open(tmp_path / "out.txt").read().splitlines()) == 2
    # the header promises more requests than the file holds: the missing ones are empty strings
    write_requests(tmp_path / "short.txt", PROMPTS[:2], count=4)
    r = run("requests", tmp_path / "short.txt", tmp_path / "out.txt", 32)
    assert r.returncode == 0 and "num requests: 4" in r.stdout
    got = [[int(t) for t in l.split()] for l in open(tmp_path / "out.txt").read().splitlines()]
    assert got == expected_tokens(PROMPTS[:2] + ["", ""], 32)
    # a line longer than a request slot (8 * (max_seq_len + 1) bytes) is cut to the slot
    write_requests(tmp_path / "long.txt", ["x" * 1000])
    r = run("requests", tmp_path / "long.txt", tmp_path / "out.txt", 4)
    assert r.returncode == 0
    assert open(tmp_path / "out.txt").read().split()[0] == str(8 * 5 - 1)
    # unreadable input
    r = run("requests", tmp_path / "absent.txt", tmp_path / "out.txt", 4)
    assert r.returncode == 3 and "cannot be opened" in r.stdout


def test_verify_output(tmp_path):
    gt = "1 2 3\n\n7\n42 43\n"
    open(tmp_path / "gt.txt", "w").write(gt)
    open(tmp_path / "same.txt", "w").write("1 2 3\n\n7\n42   43\n")              # whitespace is not significant
    r = run("verify", tmp_path / "same.txt", tmp_path / "gt.txt")
    assert r.returncode == 0 and "mismatches: 0" in r.stdout and "Total requests checked: 4" in r.stdout
    open(tmp_path / "tok.txt", "w").write("1 2 4\n\n7\n42 43\n")
    r = run("verify", tmp_path / "tok.txt", tmp_path / "gt.txt")
    assert r.returncode == 1 and "Token mismatch at position 2 (GT: 3, Generated: 4)" in r.stdout
    open(tmp_path / "len.txt", "w").write("1 2\n\n7\n42 43\n")
    r = run("verify", tmp_path / "len.txt", tmp_path / "gt.txt")
    assert r.returncode == 1 and "Length mismatch (GT: 3 tokens, Generated: 2 tokens)" in r.stdout
    open(tmp_path / "fewer.txt", "w").write("1 2 3\n\n")
    r = run("verify", tmp_path / "fewer.txt", tmp_path / "gt.txt")
    assert r.returncode == 1 and "fewer lines" in r.stdout
    open(tmp_path / "more.txt", "w").write(gt + "5\n")
    r = run("verify", tmp_path / "more.txt", tmp_path / "gt.txt")
    assert r.returncode == 1 and "more lines" in r.stdout and "mismatches: 1" in r.stdout
    r = run("verify", tmp_path / "absent.txt", tmp_path / "gt.txt")
    assert r.returncode == 255
