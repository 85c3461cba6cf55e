"""Small stand-alone hardware probes behind the design decisions of the grouped-matmul kernels.

    python -m mindspeed_amd.probes build            compile every probe for gfx950 (hipcc) into probes/bin/
    python -m mindspeed_amd.probes run NAME         run one of them on the GPU (builds it first if missing)

    mfma_power   pure MFMA loops, both bf16 shapes, random / zero operands: rate, board power, clock
    lds_rates    LDS read / write / global->LDS throughput of a compute unit by instruction form
    issue_cost   clocks of MFMA time one memory instruction of each kind costs the wavefront that issues it

None of them is used by the library; they only print tables.
"""
