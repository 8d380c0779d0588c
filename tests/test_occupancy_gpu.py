"""Occupancy probe on the device: what the compiled kernels really use against what the tile model assumes.

The reference compiles every (TH, TW, TC) candidate and records cudaOccupancyMaxActiveBlocksPerMultiprocessor for it
(2080Ti-evaluation/Gen-occupancy/template.cu:277-284); its model then reads those tables.  Here the candidates of a
layer share a few dozen kernel instantiations and the model computes occupancy in closed form from a register table,
so the probe is a test: hipFuncGetAttributes and hipOccupancyMaxActiveBlocksPerMultiprocessor for one plan of every
instantiation, compared with tdc_tile_info."""
import pytest
import torch

import tdc_amd
from tdc_amd import _lib

pytestmark = pytest.mark.gpu

DESCS = [
    tdc_amd.conv_desc(1, 64, 64, 56, 56, 3, 3, 1, 1), tdc_amd.conv_desc(1, 128, 128, 56, 56, 3, 3, 1, 1),
    tdc_amd.conv_desc(1, 256, 256, 7, 7, 3, 3, 1, 1), tdc_amd.conv_desc(1, 40, 24, 13, 13, 3, 3, 2, 1),
    tdc_amd.conv_desc(1, 256, 64, 56, 56, 1, 1, 1, 0), tdc_amd.conv_desc(1, 2048, 256, 7, 7, 1, 1, 1, 0),
    tdc_amd.conv_desc(1, 64, 128, 56, 56, 1, 1, 2, 0), tdc_amd.conv_desc(1, 3, 64, 224, 224, 7, 7, 2, 3),
]


def test_compiled_kernels_match_the_model_registers_and_occupancy():
    compiled = _lib.kernel_resources()
    seen, problems = {}, []
    for d in DESCS:
        # per kernel instantiation two candidates: the one with the most workgroups per CU by the model (its sharpest
        # occupancy claim) and the one with the largest workgroup
        dense, big = {}, {}
        for t in tdc_amd.model_enumerate(d):
            name = _lib.model_kernel_info(d, t, False)[0]
            i = tdc_amd.model_evaluate(d, t)
            if name not in dense or i.wg_per_cu > dense[name][1].wg_per_cu:
                dense[name] = (t, i)
            if name not in big or i.block_threads > big[name][1].block_threads:
                big[name] = (t, i)
        picks = [(n, "dense", v[0]) for n, v in dense.items()] + [(n, "big", v[0]) for n, v in big.items()]
        for name, kind, t in picks:
            plan = tdc_amd.Conv2dPlan(d.batch, d.C, d.N, d.H, d.W, d.KH, d.KW, d.stride, d.pad, tile=t)
            occ = plan.occupancy()
            plan.close()
            print(f"{name:52s} {kind:5s} threads {occ.block_threads:4d} lds {occ.dynamic_lds_bytes:6d}: registers "
                  f"{occ.kernel_vgprs:3d} (model {occ.model_vgprs:3d}), workgroups/CU {occ.runtime_wg_per_cu:2d} "
                  f"(model {occ.model_wg_per_cu:2d})", flush=True)
            seen[name] = occ.kernel_vgprs
            if (occ.kernel_vgprs + 7) // 8 * 8 != occ.model_vgprs:
                problems.append(f"{name}: registers per lane {occ.kernel_vgprs} vs model {occ.model_vgprs}")
            if name in compiled and occ.kernel_vgprs != compiled[name]["vgprs"] + compiled[name]["agprs"]:
                problems.append(f"{name}: runtime reports {occ.kernel_vgprs} registers, the compiler's report {compiled[name]}")
            if occ.kernel_static_lds_bytes != 0 or occ.kernel_max_threads < occ.block_threads:
                problems.append(f"{name}: static LDS {occ.kernel_static_lds_bytes}, launch bound {occ.kernel_max_threads} < {occ.block_threads}")
            # the model caps resident workgroups (8 for the staged kernels, 32 for the streamed ones); below the cap
            # it must not claim more than the runtime grants
            if occ.runtime_wg_per_cu < 1 or occ.model_wg_per_cu > occ.runtime_wg_per_cu:
                problems.append(f"{name} {t}: model claims {occ.model_wg_per_cu} workgroups per CU, runtime grants {occ.runtime_wg_per_cu}")
    assert not problems, "\n".join(problems)
    assert len(seen) >= 25, sorted(seen)
