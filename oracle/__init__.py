"""CPU oracle for the MoE context-encoding path.  TEST INFRASTRUCTURE ONLY.

This package is a numpy restatement of the numpy/torch "golden" functions that
aws-neuron/nki-library's own tests compare its kernels against.  Nothing in the
shipped library imports it: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.

Why a restatement: the reference goldens import ``nki`` / ``neuron_dtypes``
(``src/nkilib_src/nkilib/core/moe/moe_cte/moe_cte_utils.py:48-51``,
``src/nkilib_src/nkilib/core/utils/mx_torch_common.py:27-28``), which are not
installable offline, so they cannot be imported here.  The reference stores no
golden vectors (its goldens are recomputed from seeds at test time), so every
function below is pinned by closed forms, invariants, brute force on tiny
inputs and independent library routines (see ``tests/test_oracle_*.py``).

Parity unpinned (no source, fixture or mathematical fact fixes them):
  * tie / overflow behaviour of ``neuron_dtypes.static_cast`` (used for every
    fp8 / bf16 cast in the goldens; no version is pinned by the reference's
    ``pyproject.toml``).  The oracle uses round-to-nearest-even after the
    explicit saturating clip the goldens apply, i.e. IEEE/OCP behaviour.
  * hardware approximations of ``nisa.activation`` / ``nisa.quantize_mx``; the
    oracle follows the numpy goldens, not the hardware.
  * router top-k: which of several experts with equal logits ``torch.argsort``
    returns (the reference's bf16 logits tie often); the oracle selects on
    fp32 logits and breaks ties towards the lower expert index.

  * the fp8-row kind under PRE_SCALE / NO_SCALE and with clamps
    (``moe.moe_blockwise_fp8_row_ref``): the reference has no kernel with fp8
    activations on this path; the rule is the dense golden's applied to the
    row-quantised operands (the affinity scales the row's dequantisation scale).

Modules
  numerics   bf16 / fp8-e4m3fn / E8M0 encode + decode
  mx         OCP-MX (8x4 block) quantise / dequantise / matmul goldens
  blocks     token -> block index construction (bit exact, integer)
  index_ops  find_nonzero_indices / indexed_flatten / cumsum (bit exact, integer)
  rmsnorm    RMSNorm + fp8 ROW / STATIC quantise, RMSNorm -> MXFP8
  moe        blockwise MoE goldens (bf16, fp8-weight, fp8-row, MXFP8)
  router     router top-k (logits, top-k selection, affinities)
  compare    the reference comparator (max-abs-rel "maxAllClose")
"""
