"""Writes the small committed fixtures under tests/golden/ from the CPU oracle.

The reference stores no golden vectors (its goldens are recomputed from seeds at test time) and its
Python cannot be imported here (it needs the absent ``nki`` package), so these are produced by the
oracle restatement after it has been pinned by tests/test_oracle_*.py; they guard against
regressions of the oracle and of the seeded input stream.

  python tests/golden/make_fixtures.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import blocks as ob  # noqa: E402
from oracle import moe as omoe  # noqa: E402
from oracle import rmsnorm as orn  # noqa: E402
from oracle.numerics import bf16_bits  # noqa: E402


def main():
    # C1 routing (T=256, top-2, E=8, B=128): the reference's seeded router and the resulting block index
    N = ob.get_n_blocks(256, 2, 8, 128)
    mask, tp, b2e, cond = ob.generate_token_position_to_id_and_experts(256, 2, 8, 128, False, N)
    router = ob.router_with_controlled_distribution(256, 2, 8).astype(np.int32)
    np.savez_compressed(os.path.join(HERE, "c1_blocks.npz"), router=router, token_position_to_id=tp,
                        block_to_expert=b2e, conditions=cond)

    # a small MXFP8 MoE case: inputs are regenerated from the seed by tests/helpers.py, the expected output
    # (bf16 bit patterns) is stored
    from helpers import dense_case, mx_case

    c = mx_case(128, 512, 512, 4, 2, 128, seed=21)
    out = omoe.moe_blockwise_mx_ref(c["hidden"], c["aff"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"],
                                    c["tp2id"], c["b2e"], c["B"])
    c2 = dense_case(128, 256, 256, 4, 2, 128, seed=22, hidden_std=1.0)
    out2 = omoe.moe_blockwise_ref(c2["hidden"], c2["aff"], c2["gate_up_w"], c2["down_w"], c2["tp2id"], c2["b2e"],
                                  c2["B"])
    rng = np.random.default_rng(23)
    x = orn.to_bf16(rng.standard_normal((4, 1024)).astype(np.float32))
    g = orn.to_bf16(rng.random((1, 1024)).astype(np.float32))
    codes, scale = orn.rmsnorm_quant_ref(x, g, None, 0.0, False, "row")
    mxq = orn.rmsnorm_mx_quant_ref(x, g)
    np.savez_compressed(os.path.join(HERE, "small_cases.npz"), mx_out_bits=bf16_bits(out), bf16_out_bits=bf16_bits(out2),
                        row_record=orn.pack_row_record(codes, scale), mx_tok_quant=mxq["tok_quant"],
                        mx_tok_scale=mxq["tok_scale"])
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
