"""Three calls of the attention kernel on one whole 2,048-token prompt at the head
sizes of Llama 3.1 8B, and nothing else: the workload for hardware-counter runs
(`rocprofv3 --pmc ... --kernel-trace -- python3 tests/profile_attention_prefill.py`).
Not a test: pytest does not collect it."""

import math
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from mini_infer_amd import ops  # noqa: E402

DEVICE = "cuda:0"
Q_HEADS, KV_HEADS, HEAD_DIM, PAGE = 32, 8, 128, 16
TOKENS = 2048


def main() -> None:
    pages = TOKENS // PAGE
    keys = (torch.randn(pages, KV_HEADS, PAGE, HEAD_DIM, device=DEVICE) * 0.5).bfloat16()
    values = (torch.randn(pages, KV_HEADS, HEAD_DIM, PAGE, device=DEVICE) * 0.5).bfloat16()  # transposed pages
    table = torch.randperm(pages, device=DEVICE).int().view(1, pages).contiguous()
    queries = torch.randn(TOKENS, Q_HEADS * HEAD_DIM, device=DEVICE).bfloat16()
    cu = [0, TOKENS]
    positions = torch.arange(TOKENS, dtype=torch.int32, device=DEVICE)
    token_request = torch.zeros(TOKENS, dtype=torch.int32, device=DEVICE)
    cu_device = torch.tensor(cu, dtype=torch.int32, device=DEVICE)
    for _ in range(3):
        ops.paged_attention(
            queries, keys, values, table, token_request, positions, cu_device, cu,
            q_heads=Q_HEADS, kv_heads=KV_HEADS, head_dim=HEAD_DIM, scale=1 / math.sqrt(HEAD_DIM),
            window=None, max_seq_len=TOKENS, v_transposed=True,
        )
    torch.cuda.synchronize()


if __name__ == "__main__":
    main()
