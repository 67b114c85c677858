"""From a kernel's launch shape and resource use to the two profile columns the
policy reads: the compute units it can occupy and its bound class.

Counterpart of the reference's ``profiling/postprocessing/get_num_blocks.py``
(``SM_needed``, :34-52) and ``roofline_analysis.py`` (class, :37-71), restated
for a CDNA4 compute unit instead of a V100 SM:

* 4 SIMDs per CU, at most 8 resident wavefronts of 64 lanes each per SIMD;
* 512 vector registers per lane and SIMD (architectural + accumulation
  registers are one file), allocated in blocks of 8;
* 160 KiB of LDS per CU;
* at most 32 resident workgroups per CU.
"""

from math import ceil

WAVE = 64
SIMDS_PER_CU = 4
MAX_WAVES_PER_SIMD = 8
VGPRS_PER_SIMD = 512
VGPR_GRANULE = 8
LDS_PER_CU = 160 * 1024
MAX_WORKGROUPS_PER_CU = 32
TOTAL_CUS = 256                # MI355X


def workgroups_per_cu(threads_per_block, regs_per_thread=0, lds_per_block=0):
    """How many workgroups of this shape fit on one CU at once."""
    waves_per_block = max(1, ceil(threads_per_block / WAVE))
    waves_per_simd = MAX_WAVES_PER_SIMD
    if regs_per_thread > 0:
        alloc = ceil(regs_per_thread / VGPR_GRANULE) * VGPR_GRANULE
        waves_per_simd = max(1, min(MAX_WAVES_PER_SIMD, VGPRS_PER_SIMD // alloc))
    by_waves = max(1, (SIMDS_PER_CU * waves_per_simd) // waves_per_block)
    by_lds = by_waves
    if lds_per_block > 0:
        by_lds = max(1, LDS_PER_CU // lds_per_block)
    return max(1, min(by_waves, by_lds, MAX_WORKGROUPS_PER_CU))


def cu_needed(num_blocks, threads_per_block, regs_per_thread=0, lds_per_block=0):
    """``SM_needed`` for CDNA4: workgroups / resident workgroups per CU, not
    clipped to the device (the reference does not clip either)."""
    return max(1, ceil(num_blocks / workgroups_per_cu(threads_per_block,
                                                      regs_per_thread,
                                                      lds_per_block)))


COMPUTE_HINTS = ("gemm", "cijk", "conv", "igemm", "winograd", "xdlops", "mfma",
                 "attn", "fmha", "wrw", "fwd_gtc", "bwd_gtc", "implicit",
                 "naive_conv")
MEMORY_HINTS = ("elementwise", "batch_norm", "batchnorm", "bn_", "reduce", "pool",
                "copy", "fill", "softmax", "layer_norm", "layernorm", "cat",
                "index", "embedding", "dropout", "multi_tensor", "transpose",
                "add", "mul", "relu", "scatter", "gather", "nll", "sum", "triad")


def classify(name, hbm_fraction=None, mfma_fraction=None, threshold=0.6):
    """1 compute-bound, 0 memory-bound, -1 unknown.

    With hardware counters (fractions of peak HBM bandwidth and of peak matrix
    throughput, from rocprofv3) the reference's utilisation rule applies
    (roofline_analysis.py:60-66: >= 60 % decides).  Without them the kernel
    name decides, which is what the reference's op grouping amounts to for
    library ops (generate_file.py:62-86 labels cuDNN/cuBLAS ops by name)."""
    if mfma_fraction is not None and mfma_fraction >= threshold:
        return 1
    if hbm_fraction is not None and hbm_fraction >= threshold:
        return 0
    if hbm_fraction is not None and mfma_fraction is not None:
        return -1
    low = name.lower()
    if any(h in low for h in COMPUTE_HINTS):
        return 1
    if any(h in low for h in MEMORY_HINTS):
        return 0
    return -1


# MI355X peaks used to place a kernel on the roofline
PEAK_HBM_BYTES_PER_S = 8.0e12
PEAK_VECTOR_FP32_FLOPS = 157.3e12
PEAK_VECTOR_FP16_FLOPS = 314.6e12       # packed half rate
PEAK_MFMA_FP32_FLOPS = 157.3e12
PEAK_MFMA_BF16_FLOPS = 2.5e15


def classify_roofline(bytes_moved, vector_fp32_flops=0.0, vector_fp16_flops=0.0,
                      mfma_fp32_flops=0.0, mfma_bf16_flops=0.0, hbm_fraction=None,
                      mfma_fraction=None, threshold=0.6):
    """The reference's rule (profiling/postprocessing/roofline_analysis.py:37-71)
    on MI355X terms.  A kernel that executes floating-point instructions is
    compute-bound (1) when its arithmetic intensity lies right of the roofline's
    knee, else memory-bound (0); because the knee differs per instruction type
    here (matrix cores vs vector ALU), the comparison is done in time: the
    shortest time the flops could take at peak against the shortest time the
    bytes could take at peak.  A kernel without floating-point instructions falls
    back to utilisation (>= 60 % of the matrix cores -> 1, >= 60 % of HBM
    bandwidth -> 0), else unknown (-1)."""
    flops = vector_fp32_flops + vector_fp16_flops + mfma_fp32_flops + mfma_bf16_flops
    if flops > 0:
        t_compute = (vector_fp32_flops / PEAK_VECTOR_FP32_FLOPS
                     + vector_fp16_flops / PEAK_VECTOR_FP16_FLOPS
                     + mfma_fp32_flops / PEAK_MFMA_FP32_FLOPS
                     + mfma_bf16_flops / PEAK_MFMA_BF16_FLOPS)
        t_memory = bytes_moved / PEAK_HBM_BYTES_PER_S
        return 1 if t_compute > t_memory else 0
    if mfma_fraction is not None and mfma_fraction >= threshold:
        return 1
    if hbm_fraction is not None and hbm_fraction >= threshold:
        return 0
    return -1
