"""Multi-threaded CPU restatement of the reference's "recons + torch.matmul" algorithm in
torch tensor ops.  TEST INFRASTRUCTURE ONLY (checker and cpu_baseline leg of bench.py).

The reference has no CPU dequant of its own; its algorithm for every grad-mode call and every
call above 8 rows is: dequantize to a dense [K, N] buffer (quant_cuda_kernel.cu:1127-1153),
then torch.matmul (matmul_utils_4bit.py:114-127).  This file is that algorithm on CPU tensors.
Pinned bit-for-bit against q4_oracle.dequant_v2 in tests/test_oracle.py.
"""
import torch

_SHIFTS = torch.arange(0, 32, 4, dtype=torch.int32)


def dequant_v2(qweight, qzeros, scales, g_idx):
    """fp16 W [K, N] = rn16(rn16(s*q) - rn16(s*(z+1))); torch CPU half ops round once per op."""
    KW, N = qweight.shape
    G = qzeros.shape[0]
    q = ((qweight.unsqueeze(1) >> _SHIFTS.view(1, 8, 1)) & 0xF).reshape(KW * 8, N)      # :1148-1151
    z = ((qzeros.unsqueeze(2) >> _SHIFTS.view(1, 1, 8)) & 0xF).reshape(G, N)            # :1144-1147
    g = g_idx.long()
    s = scales[g]                                                                       # :1143,1146
    zero = s * (z + 1).to(torch.float16)[g]
    return s * q.to(torch.float16) - zero


def matmul_recons(x, qweight, qzeros, scales, g_idx, transpose=False):
    """matmul_utils_4bit.py:122-126 on CPU: fp16 operands, fp32 result."""
    W = dequant_v2(qweight, qzeros, scales, g_idx).float()
    return x.float() @ (W.t() if transpose else W)
