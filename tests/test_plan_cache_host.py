"""The plan cache's slot state machine (torchopt_amd/csrc/plan_cache.hpp) on the CPU: the C++
test in tests/host/ drives it with a fake backend that models launches in flight, events and
blocking frees -- least-recently-used eviction per stream, memory a slot outgrows parked until
its readers are done, a full table taking over the oldest slot of another stream through a
blocking free, remembered calls, allocation failure, and four host threads sharing one stream
with more lists than slots (nobody may take a slot between another thread's fill and launch)."""

from __future__ import annotations

import os
import shutil
import subprocess

import pytest

from conftest import REPO


@pytest.mark.skipif(shutil.which('g++') is None, reason='needs g++')
def test_plan_cache_state_machine(tmp_path):
    exe = tmp_path / 'plan_cache_test'
    subprocess.run(['g++', '-O1', '-std=c++17', '-pthread', '-Wall', '-Werror',
                    '-I', os.path.join(REPO, 'torchopt_amd', 'csrc'),
                    os.path.join(REPO, 'tests', 'host', 'plan_cache_test.cpp'), '-o', str(exe)],
                   check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip() == 'ok', run.stdout + run.stderr
