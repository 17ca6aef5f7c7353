"""What the compiler made of the library's kernels, read from the built code objects' metadata
(no GPU needed): a kernel whose registers spill to scratch memory reloads them inside its loops,
behind the weight stream's loads, and loses microseconds without failing any parity test.  The
streamed families (loader waves + arithmetic waves) budget 168 registers a wave; this pins that
none of them spills, and that a wave's register count lets the launch shape be resident."""
import pytest

from gllm_amd.code_objects import all_kernels

# kernels known to spill, with the most scratch bytes per lane they may use: 64-row tiles of the
# fetch-and-compute GEMM for Q6_K and Q8_0 (two accumulator tiles a wave), and a variant of the
# chained launch that only runs under option "chain_dependent"
KNOWN_SCRATCH = {"gq_mmf_q6k_t2": 64, "gq_mmf_q8_0_t2": 256, "gq_mmf_q8_0_t2_bf16": 256, "gq_mm8c_q5k_f_d": 64}


@pytest.fixture(scope="module")
def kernels():
    found = all_kernels()
    if not found:
        pytest.skip("no built code objects (python -m gllm_amd.build)")
    return found


def test_every_unit_is_there(kernels):
    from gllm_amd.build import KERNEL_UNITS
    assert {k["unit"] for k in kernels.values()} == set(KERNEL_UNITS)
    for name in ("gq_mm8s_q4k_p1_e1_a", "gq_mm8c_q4k_f", "gq_mmfr_q4k", "gq_mmfs_q4k", "gq_moe_mm8s_q6k", "gq_finish_elem", "gq_touch"):
        assert name in kernels, name


def test_no_kernel_spills_unnoticed(kernels):
    bad = {n: k["scratch_bytes"] for n, k in kernels.items() if k["scratch_bytes"] > KNOWN_SCRATCH.get(n, 0)}
    assert not bad, f"kernels with scratch (spilled registers): {bad}"


def test_registers_fit_the_launch_shape(kernels):
    # a SIMD holds 512 registers per lane; waves of a workgroup are dealt to the CU's four SIMDs
    for name, k in kernels.items():
        waves = (k["max_threads"] + 63) // 64
        per_simd = (waves + 3) // 4
        regs = ((k["vgprs"] + k["agprs"] + 7) // 8) * 8
        assert per_simd * regs <= 512, f"{name}: {waves} waves of {regs} registers do not fit a CU"
