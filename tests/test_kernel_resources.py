"""The compiler's own figures for every kernel of the library (registers, scratch memory per lane, occupancy), as
`python -m cntk_amd.build` leaves them beside the object files: no kernel may spill more than a few registers' worth.

A kernel whose register budget (`amdgpu_waves_per_eu`) is a little too small still compiles and still gives the right
bytes, only many times slower -- the table-driven stripe reduction at six pieces per thread once ran 6144-row stripes in
548 us instead of 39 us on 388 bytes of scratch per lane -- so the bound is checked where it costs nothing."""
import os

import pytest

from cntk_amd import build

# the largest scratch of a kernel today: the tall stripe reductions at 25 pieces per thread (80001 to 102400 rows), which
# have the SIMD's registers to themselves and still keep 79 values too many
MAX_SCRATCH_BYTES_PER_LANE = 160


def read_report(source):
    path = build.resource_report_path(source)
    if not os.path.exists(path):
        pytest.skip("no resource report at %s: build the library first (python -m cntk_amd.build)" % path)
    kernels = []
    with open(path) as f:
        for line in f:
            kernels.append(dict(kv.split("=", 1) for kv in line.split()))
    return kernels


def all_kernels(sources):
    return [k for source in sources for k in read_report(source)]


FLOAT_SOURCES = [s for s in build.SOURCES if not s.endswith("_f64.hip")]


@pytest.mark.parametrize("sources", [FLOAT_SOURCES, ["quantizer_api_f64.hip"]], ids=["float", "double"])
def test_no_kernel_lives_on_scratch_memory(sources):
    kernels = all_kernels(sources)
    assert len(kernels) > 100, "the reports of %s list %d kernels only" % (sources, len(kernels))
    worst = sorted(kernels, key=lambda k: -int(k["ScratchSize"]))[:5]
    print([(k["name"][:70], k["ScratchSize"], k["VGPRs"]) for k in worst])
    for k in kernels:
        assert int(k["ScratchSize"]) <= MAX_SCRATCH_BYTES_PER_LANE, \
            "%s: %s bytes of scratch per lane (%s registers spilled at %s registers, %s wavefronts per SIMD)" % (
                k["name"], k["ScratchSize"], k["VGPRsSpill"], k["VGPRs"], k["Occupancy"])


def test_headline_kernels_spill_nothing():
    """The kernels of the headline benchmark and of the batched launches: no scratch at all."""
    kernels = all_kernels(FLOAT_SOURCES)
    seen = 0
    for k in kernels:
        n = k["name"]
        if any(s in n for s in ("quantize_col_kernel", "quantize_batch_kernel", "stripe_reduce_col_kernel", "stripe_reduce_batch_kernel",
                                "unquantize_kernel", "unquantize_batch_kernel", "stripe_reduce_lut_kernelILb0ELi6E", "stripe_reduce_lut_kernelILb1ELi6E")):
            seen += 1
            assert int(k["ScratchSize"]) == 0, "%s uses %s bytes of scratch per lane" % (n, k["ScratchSize"])
    assert seen >= 20


def wavefronts_by_scalar_registers(sgprs):
    """Resident wavefronts per SIMD that a kernel's scalar registers allow on the MI355X as it runs here: every wavefront
    is given 16 scalar registers beyond its kernel's own, in blocks of 16, out of 800 per SIMD (measured with a kernel that
    only holds registers: up to 80 -> 8 wavefronts, up to 96 -> 7, beyond -> 6). The compiler's occupancy figure does not
    count those 16."""
    return min(8, 800 // ((sgprs + 15) // 16 * 16 + 16))


@pytest.mark.parametrize("sources", [FLOAT_SOURCES, ["quantizer_api_f64.hip"]], ids=["float", "double"])
def test_scalar_registers_cost_the_stripe_kernels_no_wavefront(sources):
    """The kernels that take a set of stripes by value are the ones that reach 80 scalar registers; they are built with a
    cap, so the wavefronts that their vector registers allow are the ones that run."""
    seen = 0
    for k in all_kernels(sources):
        n = k["name"]
        if any(s in n for s in ("stripe_reduce_colg_kernel", "stripe_reduce_batch_kernel", "stripe_reduce_tile_kernel")):
            seen += 1
            assert wavefronts_by_scalar_registers(int(k["SGPRs"])) >= int(k["Occupancy"]), \
                "%s: %s scalar registers allow %d wavefronts per SIMD, its vector registers %s" % (
                    n, k["SGPRs"], wavefronts_by_scalar_registers(int(k["SGPRs"])), k["Occupancy"])
    assert seen >= 8


def test_kernels_that_address_lds_by_number_declare_none_of_their_own():
    """The multi-bit column stripe reduction reads its decoding tables and writes its column at LDS addresses counted from 0
    (`lds_read` / `lds_write`), which is where a kernel's LDS from the launch starts only if the kernel declares none
    itself: the compiler's figure for declared LDS must be 0 for every kernel that contains that body."""
    seen = 0
    for k in all_kernels(FLOAT_SOURCES):
        n = k["name"]
        if "stripe_reduce_colg_kernel" in n or "stripe_reduce_batch" in n:
            seen += 1
            assert int(k["LDS"]) == 0, "%s declares %s bytes of LDS of its own" % (n, k["LDS"])
    assert seen >= 10
