"""One stateful-model GEMM (ops/hip_seq.py matmul_nt, bf16) launched a few times: the target of
rocprofv3 --pmc counter passes (summarised by scripts/pmc_summary.py).

    python scripts/seq_gemm_one.py M N K [launches]
"""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from flexible_llm_sharding_amd.ops import get_ops  # noqa: E402

M, N, K = (int(x) for x in sys.argv[1:4])
n = int(sys.argv[4]) if len(sys.argv) > 4 else 5
dev = torch.device("cuda", 0)
ops = get_ops(dev, torch.bfloat16, family="hybrid")
a = torch.randn(M, K, device=dev).to(torch.bfloat16)
w = (0.02 * torch.randn(N, K, device=dev)).to(torch.bfloat16)
for _ in range(n):
    c = ops.matmul_nt(a, w)
torch.cuda.synchronize()
print("ok", tuple(c.shape))
