"""The benchmark's own configurations run end to end (few steps, no CPU leg) and report a
plausible line: keeps bench.py in step with the C ABI."""

from __future__ import annotations

import json

import pytest
import torch

import bench

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('cfg', sorted(bench.CONFIGS))
def test_bench_config_runs(cfg, capsys):
    assert torch.cuda.is_available()
    assert bench.main(['--config', str(cfg), '--steps', '3', '--warmup', '1',
                       '--no-cpu-baseline']) == 0
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert line['n_gpus'] == 1 and line['steps'] == 3 and line['unit'] == 'elements/s'
    assert line['value'] > 0 and line['ms_per_step'] > 0
    assert line['config']['workload'] == bench.CONFIGS[cfg]['name']
    roof = line['roofline']
    assert roof['bound'] == 'hbm' and roof['peak'] == 8000.0 and roof['unit'] == 'GB/s'
    assert roof['achieved'] > 0 and roof['frac'] > 0
    torch.cuda.empty_cache()


@pytest.mark.parametrize('state', ['init', 'separate', 'plain'])
def test_bench_state_allocation_modes(state, capsys):
    """The three ways the benchmark can allocate the moments (as the package's init does, each in a
    block of its own at the preferred phase, or wherever the allocator puts them)."""
    assert bench.main(['--config', '0', '--steps', '2', '--warmup', '1', '--no-cpu-baseline',
                       '--state', state]) == 0
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert line['config']['state_allocation'] == state
    phases = line['config']['address_mod_16KiB']
    assert (phases['mu'], phases['nu']) == ((0, 0) if state == 'plain' else (8192, 0))
    torch.cuda.empty_cache()


def test_bench_refuses_more_than_one_gpu(capsys):
    assert bench.main(['--gpus', '2']) == 2
    assert 'one GPU' in capsys.readouterr().err


def test_ceiling_probe_runs():
    """The arithmetic-free probes behind `bench.py --ceiling`, on small arrays."""
    out = bench.run_ceiling(array_bytes=1 << 26, reps=3)
    assert out['unit'] == 'GB/s' and out['peak'] == 8000.0
    assert {'3R0W', '0R3W', '1R1W', '3R3W', '3R3W in place', '4R3W in place'} <= set(out['ceilings'])
    for row in out['ceilings'].values():
        assert row['GB/s'] > 0 and row['waves_per_cu'] in bench.RESIDENCY_LEVELS
    torch.cuda.empty_cache()


def test_placement_sweep_runs():
    """The operator over placements of its arrays inside one allocation (`bench.py --placements`),
    on small arrays and a short ladder."""
    out = bench.run_placements(reps=2, n=1 << 22, ladder=(0, 8, 64))
    assert out['placements'] == 6 and out['unit'] == 'GB/s'
    assert 0 < out['min'] <= out['median'] <= out['max']
    assert set(out['GB/s_by_placement']) == {'mu +0 KiB', 'mu +8 KiB', 'mu +64 KiB'}
    torch.cuda.empty_cache()


def test_state_phase_sweep_runs():
    """The operator on separate allocations with the moments at a grid of phases
    (`bench.py --state-phases`), on small arrays and a coarse grid."""
    out = bench.run_state_phases(reps=2, n=1 << 22, step_kib=8, span_kib=16)
    assert out['unit'] == 'GB/s' and out['library_phases_kib'] == {'mu': 8, 'nu': 0}
    assert set(out['GB/s_by_phase']) == {'mu +0 KiB', 'mu +8 KiB'}
    assert out['at_library_phases'] == out['GB/s_by_phase']['mu +8 KiB']['nu +0 KiB'] > 0
    assert len(out['unshifted_after_each_row']) == 2
    torch.cuda.empty_cache()


def test_state_distance_sweep_runs():
    """The operator with both moments in one block over a ladder of distances
    (`bench.py --state-distances`), on small arrays and a short ladder."""
    out = bench.run_state_distances(reps=2, n=1 << 22, distances_mib=(0, 1, 8))
    assert out['unit'] == 'GB/s' and len(out['GB/s_by_distance_beyond_the_array_size']) == 2
    assert set(out['GB/s_by_distance_beyond_the_array_size'][0]) == {'0 MiB', '1 MiB', '8 MiB'}
    assert out['blocks_of_their_own_at_their_phases'] > 0 and out['allocator_placement'] > 0
    assert len(out['GB/s_by_phases_of_the_moments_and_of_the_gradient']) == 4
    torch.cuda.empty_cache()
