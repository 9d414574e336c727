"""What the compiler made of the kernels, read from the metadata of the built library's own code
object (no GPU needed): the launch arithmetic of the host side assumes single-wave workgroups of
64 lanes whose residency is bounded by the dynamic-LDS reservation alone, so a kernel must use no
static LDS (one that does loses a residency level: an op struct the compiler kept in memory once
cost the float16 step 7 % that way), no scratch memory and no spilled registers, and the
whole-tile kernels must fit the highest residency level in registers."""

from __future__ import annotations

import os
import re
import shutil
import subprocess

import pytest

from conftest import REPO

LLVM = '/opt/rocm/llvm/bin'
TOOLS = [os.path.join(LLVM, t) for t in ('llvm-objcopy', 'clang-offload-bundler', 'llvm-readelf')]
LIB = os.path.join(REPO, 'torchopt_amd', 'libtoa_adam.so')


@pytest.fixture(scope='module')
def code_object(tmp_path_factory):
    """The gfx950 code object inside the built library, unbundled into a file of its own."""
    if not all(os.path.exists(t) for t in TOOLS):
        pytest.skip('needs the LLVM tools of ROCm')
    if not os.path.exists(LIB):
        pytest.skip('libtoa_adam.so is not built')
    tmp = tmp_path_factory.mktemp('code_object')
    fatbin, code = str(tmp / 'fatbin'), str(tmp / 'gfx950.co')
    subprocess.run([TOOLS[0], '--dump-section', f'.hip_fatbin={fatbin}', LIB, os.devnull],
                   check=True)
    subprocess.run([TOOLS[1], '--unbundle', '--type=o', f'--input={fatbin}',
                    '--targets=hipv4-amdgcn-amd-amdhsa--gfx950', f'--output={code}'], check=True)
    return code


@pytest.fixture(scope='module')
def kernels(code_object):
    notes = subprocess.run([TOOLS[2], '--notes', code_object], check=True, capture_output=True,
                           text=True).stdout
    # one block per kernel, opened by "  - .first_key:"; the kernel's own keys are indented by
    # four spaces (those of its arguments deeper), in alphabetical order, `.name` among them
    found, current = {}, None
    for line in notes.splitlines():
        m = re.match(r'(  - |    )\.(\w+):\s*(\S*)\s*$', line)
        if not m:
            continue
        opener, key, value = m.groups()
        if opener == '  - ':
            current = {}
        if current is None:
            continue
        if key == 'name':
            found[value] = current
        elif value.lstrip('-').isdigit():
            current[key] = int(value)
    demangle = shutil.which('c++filt')
    if demangle:
        names = subprocess.run([demangle], input='\n'.join(found), capture_output=True,
                               text=True).stdout.splitlines()
        found = dict(zip(names, found.values()))
    return found


def test_every_kernel_is_there_and_none_uses_static_lds_scratch_or_spills(kernels):
    assert len(kernels) > 300  # every op x element type x kernel shape
    streaming = 0
    for name, k in kernels.items():
        assert k['wavefront_size'] == 64, name
        assert k['group_segment_fixed_size'] == 0, f'static LDS in {name}'
        assert k['private_segment_fixed_size'] == 0, f'scratch memory in {name}'
        assert k['sgpr_spill_count'] == 0 and k['vgpr_spill_count'] == 0, f'spills in {name}'
        if 'stream_kernel' in name or 'full_tiles_kernel' in name:
            streaming += 1
            assert k['max_flat_workgroup_size'] == 64, f'{name}: one wave per workgroup'
            assert k['vgpr_count'] <= 128, f'{name}: fewer than 16 waves per CU fit'
    assert streaming > 300


def test_whole_tile_kernels_fit_every_residency_level(kernels):
    whole = {n: k for n, k in kernels.items() if 'full_tiles_kernel' in n}
    if not whole:
        pytest.skip('kernel names could not be demangled')
    for name, k in whole.items():
        assert k['vgpr_count'] <= 64, f'{name}: {k["vgpr_count"]} VGPRs, 32 waves per CU need 64'


def test_no_packed_float32_arithmetic_and_no_fused_half_arithmetic(code_object):
    """The library is built with packed float32 code generation off (some forms of
    v_pk_add_f32 / v_pk_mul_f32 / v_pk_fma_f32 have given wrong results on this hardware) and
    without contraction (every product and sum rounds on its own: no fused multiply-add may
    appear in the packed half arithmetic of the float16 kernels either)."""
    objdump = os.path.join(LLVM, 'llvm-objdump')
    if not os.path.exists(objdump):
        pytest.skip('needs llvm-objdump')
    text = subprocess.run([objdump, '-d', '--no-show-raw-insn', code_object], check=True,
                          capture_output=True, text=True).stdout
    assert 'v_pk_mul_f16' in text and 'v_pk_add_f16' in text  # the float16 pairs are there
    for banned in ('v_pk_add_f32', 'v_pk_mul_f32', 'v_pk_fma_f32', 'v_pk_fma_f16',
                   'v_pk_mad_f16'):
        assert banned not in text, banned
