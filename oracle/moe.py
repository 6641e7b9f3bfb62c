"""moe_align_block_size and the block-FP8 fused MoE, restated from the reference (CPU)."""
import numpy as np
import torch

from .gemm import block_fp8_matmul, block_int8_matmul
from .quant import group_quant


def max_num_tokens_padded(numel: int, num_experts: int, block_size: int) -> int:
    """Size of sorted_token_ids chosen by the wrapper,
    python/sglang/srt/layers/moe/moe_runner/triton_utils/moe_align_block_size.py:60-63."""
    if numel < num_experts + 1:
        return numel * block_size
    return numel + (num_experts + 1) * (block_size - 1)


def moe_align_block_size(topk_ids: np.ndarray, num_experts: int, block_size: int, max_padded: int,
                         pad_sorted_token_ids: bool = True):
    """sgl-kernel/csrc/moe/moe_align_kernel.cu:27-41 (scatter), :55-233 (count, padded
    prefix, expert_ids by binary search).  `num_experts` is the operator's argument, i.e.
    the number of buckets: bucket b holds ids equal to b-1, bucket 0 the filtered id -1.
    Slots inside one expert's span are filled in ascending flat index (the reference's
    order there depends on atomics; its test compares spans as sets).
    Returns (sorted_ids[max_padded] int32, expert_ids[ceil(max_padded/bs)] int32 with only
    the first post_pad/bs entries meaningful (others -2 here), post_pad int, cumsum int32[num_experts+1])."""
    flat = np.asarray(topk_ids).reshape(-1).astype(np.int64)
    numel = flat.size
    bucket = flat + 1
    cnt = np.bincount(bucket, minlength=num_experts)[:num_experts]
    padded = (cnt + block_size - 1) // block_size * block_size
    prefix = np.zeros(num_experts + 1, dtype=np.int64)
    prefix[1:] = np.cumsum(padded)
    post_pad = int(prefix[-1])
    sorted_ids = np.full(max_padded, numel if pad_sorted_token_ids else -1, dtype=np.int32)
    fill = prefix[:-1].copy()
    for i in range(numel):
        b = bucket[i]
        sorted_ids[fill[b]] = i
        fill[b] += 1
    nblk = -(-max_padded // block_size)
    expert_ids = np.full(nblk, -2, dtype=np.int32)
    for j in range(post_pad // block_size):
        start = j * block_size
        b = int(np.searchsorted(prefix[:num_experts], start, side="right")) - 1  # first prefix > start, minus one
        expert_ids[j] = b - 1
    return sorted_ids, expert_ids, post_pad, fill.astype(np.int32)


def topk_softmax(logits: torch.Tensor, topk: int, renormalize: bool = True, moe_softcapping: float = 0.0,
                 correction_bias: torch.Tensor = None):
    """fused_topk_torch_native, python/sglang/srt/layers/moe/topk.py:550-588: fp32 softmax,
    torch.topk, optional renormalisation.  Returns (weights fp32 [M,topk], ids int32).
    moe_softcapping / correction_bias transform the logits first as the operator does
    (sgl-kernel/csrc/moe/moe_topk_softmax_kernels.cu:108-115: tanh(x/c)*c, then + bias[e]); ties between equal
    probabilities go to the lower expert index (:540-548), which a stable descending sort reproduces."""
    x = logits.to(torch.float32)
    if moe_softcapping:
        x = torch.tanh(x / moe_softcapping) * moe_softcapping
    if correction_bias is not None:
        x = x + correction_bias.to(torch.float32)
    p = torch.softmax(x, dim=-1)
    order = torch.sort(p, dim=-1, descending=True, stable=True).indices[:, :topk]
    w, ids = torch.gather(p, 1, order), order
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    return w.to(torch.float32), ids.to(torch.int32)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """silu in fp32, rounded to the storage dtype, then multiplied by the second half in the
    storage dtype (sgl-kernel/csrc/elementwise/activation.cu:55-58,82-101; equals
    SiluAndMul.forward_native = F.silu(x[:d]) * x[d:] on bf16 tensors)."""
    d = x.shape[-1] // 2
    g = x[..., :d].to(torch.float32)
    s = (g / (1.0 + torch.exp(-g))).to(x.dtype)
    return s * x[..., d:]


def fused_moe_block_fp8(x: torch.Tensor, w13_q: np.ndarray, w2_q: np.ndarray, w13_s: np.ndarray,
                        w2_s: np.ndarray, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                        block=(128, 128), routed_scaling_factor: float = 1.0, quant_form: str = "divide",
                        int8: bool = False):
    """int8=True is the block-INT8 twin (torch_w8a8_block_int8_moe, test/registered/quant/test_block_int8.py:101-131):
    int8 weights, activations group-quantised to int8, block_int8_matmul in place of block_fp8_matmul.
    Block-FP8 fused MoE: per (token, k): h = bf16(blockgemm(q(x), w13[e])); a = silu(h[:I])*h[I:];
    y = bf16(blockgemm(q(a), w2[e]) * w[t,k]); out[t] = bf16(rsf * sum_k f32(y)).
    torch_w8a8_block_fp8_moe, test/manual/quant/test_block_fp8.py:518-547, with the weight
    applied on the fp32 accumulator and the fp32 top-k sum of the fused kernels
    (fused_moe_triton_kernels.py:602-606,1084-1099).
    w13_q [E, 2I, H] codes, w2_q [E, H, I] codes, scales [E, nb, kb]."""
    m, h = x.shape
    topk = topk_ids.shape[1]
    ids = topk_ids.reshape(-1).numpy()
    xa = x.view(m, 1, h).repeat(1, topk, 1).reshape(-1, h)
    dst = "int8" if int8 else "fp8"
    mm = block_int8_matmul if int8 else block_fp8_matmul
    xq, xs, _ = group_quant(xa, block[1], form=quant_form, dst=dst)
    hidden_out = w2_q.shape[1]
    y = torch.zeros(m * topk, hidden_out, dtype=torch.float32)
    w_flat = topk_weights.reshape(-1).to(torch.float32)
    for e in np.unique(ids):
        if e < 0:
            continue
        sel = np.nonzero(ids == e)[0]
        inter = mm(xq[sel], w13_q[e], xs[sel], w13_s[e], block, out_dtype=x.dtype)
        act = silu_and_mul(inter)
        aq, a_s, _ = group_quant(act, block[1], form=quant_form, dst=dst)
        o = mm(aq, w2_q[e], a_s, w2_s[e], block, return_fp32=True)
        y[sel] = (o * w_flat[sel].view(-1, 1)).to(x.dtype).to(torch.float32)
    out = (y.view(m, topk, hidden_out).sum(dim=1) * routed_scaling_factor).to(x.dtype)
    return out
