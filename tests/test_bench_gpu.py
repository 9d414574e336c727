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
    assert roof['achieved'] > 0 and roof['frac'] > 0 and roof['frac_by_wall_clock'] > 0
    beside = line['beside_the_headline']
    if cfg in (2, 3):  # large single tensors: every leg beside the headline
        assert {'cold_start', 'clock', 'state_where_the_allocator_puts_it',
                'one_launch_per_iteration_between_other_work'} <= set(beside)
        cold = beside['cold_start']
        assert cold['frac'] > 0 and len(cold['shader_MHz_beside_the_timed_steps']) >= 1
        assert beside['state_where_the_allocator_puts_it']['address_mod_16KiB'] == {
            'updates': 0, 'mu': 0, 'nu': 0}
        assert line['config']['load_order_kept_for_this_call_site'] in (-1, 0, 1, 2, 3)
    if cfg >= 2:  # bandwidth-bound: clock evidence and the one-launch-per-iteration leg
        probes = beside['clock']['probes']
        assert 300 < probes['before_the_timed_region']['shader_MHz'] < 4000
        assert 300 < probes['after_the_timed_region']['shader_MHz'] < 4000
        assert beside['clock']['shader_MHz_beside_the_per_step_pass']
        situ = beside['one_launch_per_iteration_between_other_work']
        assert situ['iterations'] == 50 and situ['other_work_ms_per_iteration'] >= 5.0
        assert 0 < situ['operator_ms_min'] <= situ['operator_ms_median'] <= situ['operator_ms_max']
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
