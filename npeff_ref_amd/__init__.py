"""MI355X-native D-NPEFF NMF hot path.

The product is ``lib/libdnpeff_hip.so`` (hand-written HIP kernels for gfx950
behind the C ABI of ``include/dnpeff.h``) and the two C++ executables under
``csrc/host``.  This package is the thin ctypes binding used by the tests and
by ``bench.py``; it mirrors the reference's driver classes
(``MuNmf`` -- cc/cuda_d_npeff/src/nmf/sparse/multi_mu_dense_factors_nmf1.h:81-274,
``Learner`` -- cc/cuda_d_npeff/src/nmf/sparse2/nmf_sparse_H.h:42-345).

There is no CPU fallback: importing :mod:`npeff_ref_amd.binding` raises if the
library has not been built.
"""

from .binding import (  # noqa: F401
    DnpeffError,
    Csr,
    DeviceArray,
    MuNmf,
    MuNmfParams,
    Learner,
    LearnerParams,
    lib,
    device_count,
    size_of_split,
    uniform_at,
    synth_pef_host,
    synth_pef_host_rows,
    gather_rows,
    KERNEL_CLASSES,
    sync,
    device_info,
    device_memory,
    plan_estimate,
    tuning_set,
    tuning_get,
    tuning_reset,
    op_mu,
    op_sparsify_columns,
    op_spmm_n,
    op_threshold_compact,
    topk_rows,
    op_spmm_t,
    op_gram,
    op_gram_static,
    op_xg_mu,
    op_xg_mu_gram,
    op_dot,
    op_spsp_dense,
    op_init_uniform,
)
