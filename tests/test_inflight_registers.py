"""The compiled code of the resident-activation weight-streaming kernels must not touch a register whose asm-issued
load may still be in flight (ajllm_amd/asm_check.py).  Runs without a GPU: hipcc cross-compiles a handful of
instantiations to gfx950 assembly (a few seconds) and the listing is scanned."""

import shutil

import pytest

from ajllm_amd import asm_check

SOURCE = """
#include <hip/hip_runtime.h>
#include "ajq_common.h"
#include "skinny_resident_kernels.h"
namespace ajq {
#define PLAIN const u32x4_t*, const uint32_t*, const uint16_t*, int, int, int, void*, int, const uint16_t*
template __global__ void dequant_skinny_resident_kernel<4, 8, false, 2>(PLAIN);
template __global__ void dequant_skinny_resident_kernel<4, 1, true, 2>(PLAIN);
template __global__ void dequant_skinny_resident_kernel<4, 4, true, 1>(PLAIN);
template __global__ void dequant_skinny_resident_kernel<2, 16, false, 1>(PLAIN);
template __global__ void dequant_skinny_resident_epi_kernel<4, 8, false, 4, 2>(PLAIN, GemvEpilogue);
template __global__ void dequant_skinny_resident_epi_kernel<2, 3, true, 5, 1>(PLAIN, GemvEpilogue);
template __global__ void dequant_skinny_resident_split_kernel<4, 4, true, 1, 7>(PLAIN, SkinnySplit);
template __global__ void dequant_skinny_resident_split_epi_kernel<4, 4, false, 2, 1, 7>(PLAIN, GemvEpilogue, SkinnySplit);
}
"""


# the tile GEMMs keep asm-issued weight loads in flight around their main loops (one linear pass over each loop body)
TILE_SOURCE = """
#include <hip/hip_runtime.h>
#include "ajq_common.h"
#include "gemm_kernels.h"
#include "gemm_ring_kernels.h"
#include "gemm_split_kernels.h"
#include "gemm_wide_kernels.h"
namespace ajq {
#define TILE const uint16_t*, int, int, const u32x4_t*, const uint32_t*, const uint16_t*, int, void*, int
template __global__ void dequant_gemm256w_kernel<false, false>(TILE);
template __global__ void dequant_gemm256w_kernel<true, true>(TILE);
template __global__ void dequant_gemm256s_kernel<true, false>(TILE);
template __global__ void dequant_gemm256r_w8_kernel<false>(const uint16_t*, int, int, const u32x4_t*, const uint16_t*, int, void*, int);
}
"""


def test_the_scan_flags_a_copy_between_a_load_and_its_wait():
    listing = """
_Z3badv:
	global_load_dwordx4 v[2:5], v1, s[0:1]
	global_load_dwordx4 v[6:9], v1, s[2:3]
	s_waitcnt vmcnt(1)
	v_mov_b32_e32 v10, v3
	v_mov_b32_e32 v11, v7
	s_waitcnt vmcnt(0)
	v_add_u32_e32 v12, v6, v9
	s_endpgm
_Z4goodv:
	global_load_dwordx4 v[2:5], v1, s[0:1]
	v_mov_b32_e32 v10, v1
	s_waitcnt vmcnt(0)
	v_mov_b32_e32 v11, v2
	global_load_lds_dwordx4 v1, s[0:1]
	global_store_dword v1, v11, s[0:1]
	s_endpgm
"""
    found = asm_check.scan(listing)
    assert list(found) == ["_Z3badv", "_Z4goodv"]
    assert len(found["_Z3badv"]) == 1 and "v11, v7" in found["_Z3badv"][0]  # v3 had landed, v7 had not
    assert found["_Z4goodv"] == []


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_resident_kernels_leave_registers_of_loads_in_flight_alone():
    found = asm_check.scan(asm_check.compile_device_asm(SOURCE), "dequant_skinny_resident")
    assert len(found) == 8, sorted(found)
    offending = {name: lines[:3] for name, lines in found.items() if lines}
    assert not offending, offending


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_tile_gemm_kernels_leave_registers_of_loads_in_flight_alone():
    found = asm_check.scan(asm_check.compile_device_asm(TILE_SOURCE), "dequant_gemm256")
    assert len(found) == 4, sorted(found)
    offending = {name: lines[:3] for name, lines in found.items() if lines}
    assert not offending, offending
