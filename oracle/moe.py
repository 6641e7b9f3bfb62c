"""moe_align_block_size and the block-FP8 fused MoE, restated from the reference (CPU).

Test infrastructure: only the tests, the smoke check and the CPU-baseline leg of the benchmark import this module.
Parity unpinned: moe_activation's gemm1_alpha / gemm1_limit forms restate torch.compile'd helpers as "fp32, rounded
once"; the reference holds no fixture for them (pinned only by their reduction to F.silu at an infinite limit and by
hand-made clamp cases)."""
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


def topk_sigmoid(logits: torch.Tensor, topk: int, renormalize: bool = False, correction_bias: torch.Tensor = None):
    """torch_topk_sigmoid_native, sgl-kernel/benchmark/bench_moe_topk_sigmoid.py:31-51 (the model the reference's
    own test compares with, sgl-kernel/tests/test_moe_topk_sigmoid.py:47-58): fp32 sigmoid, the k largest
    score + bias, weights = the chosen scores (the kernel writes (score + bias) - bias,
    sgl-kernel/csrc/moe/moe_topk_sigmoid_kernels.cu:340-346, which is what is restated here), optional division by
    their sum.  Equal values pick the lower expert index (:325-330): a stable descending sort."""
    x = logits.to(torch.float32)
    s = 1.0 / (1.0 + torch.exp(-x))
    choice = s if correction_bias is None else s + correction_bias.to(torch.float32)
    order = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :topk]
    w = torch.gather(choice, 1, order)
    if correction_bias is not None:
        w = w - correction_bias.to(torch.float32)[order]
    if renormalize:
        w = w * (1.0 / w.sum(dim=-1, keepdim=True))
    return w.to(torch.float32), order.to(torch.int32)


def _act_f32(g: torch.Tensor, activation: str) -> torch.Tensor:
    """The three activations of sgl-kernel/csrc/elementwise/activation.cu:55-83 on fp32 values."""
    if activation == "silu":
        return g / (1.0 + torch.exp(-g))
    if activation == "gelu":
        return g * (0.5 * (1.0 + torch.erf(g * 0.7071067811865476)))
    if activation == "gelu_tanh":
        return g * (0.5 * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g))))
    raise ValueError(activation)


def act_and_mul(x: torch.Tensor, activation: str) -> torch.Tensor:
    """The activation in fp32, rounded to the storage dtype, then multiplied by the second half in the storage
    dtype (act_and_mul_kernel, sgl-kernel/include/hip/hip_act_and_mul.cuh:29-56, with the functions of
    sgl-kernel/csrc/elementwise/activation.cu:55-83)."""
    d = x.shape[-1] // 2
    s = _act_f32(x[..., :d].to(torch.float32), activation).to(x.dtype)
    return s * x[..., d:]


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """silu in fp32, rounded to the storage dtype, then multiplied by the second half in the
    storage dtype (sgl-kernel/csrc/elementwise/activation.cu:55-58,82-101; equals
    SiluAndMul.forward_native = F.silu(x[:d]) * x[d:] on bf16 tensors)."""
    return act_and_mul(x, "silu")


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """sgl-kernel/csrc/elementwise/activation.cu:62-67,129-149."""
    return act_and_mul(x, "gelu")


def gelu_tanh_and_mul(x: torch.Tensor) -> torch.Tensor:
    """sgl-kernel/csrc/elementwise/activation.cu:76-83,107-127."""
    return act_and_mul(x, "gelu_tanh")


def moe_activation(h: torch.Tensor, activation: str = "silu", is_gated: bool = True, gemm1_alpha: float = None,
                   gemm1_limit: float = None, swiglu_limit: float = None) -> torch.Tensor:
    """What fused_experts_impl puts between its two GEMMs
    (python/sglang/srt/layers/moe/moe_runner/triton_utils/fused_moe.py:530-647): the gated forms above, or the plain
    activation of the whole row (F.silu, F.gelu, relu squared) when the layer is not gated.  Gated SiLU has three
    clamped variants: gemm1_alpha (GPT-OSS: gate and up interleaved, gate * sigmoid(alpha * gate) * (up + 1) on
    clamped values, :324-331), gemm1_limit alone (silu(gate) clamped from above times clamped up, :315-321) -- both
    are torch.compile'd pointwise functions there, i.e. evaluated in fp32 and rounded once -- and swiglu_limit (gate
    clamped from above, up from both sides, in the storage dtype, then silu_and_mul, :565-569,580)."""
    if is_gated and activation == "silu":
        if gemm1_alpha is not None:
            assert gemm1_limit is not None
            gate, up = h[..., ::2].float(), h[..., 1::2].float()
            gate = gate.clamp(max=gemm1_limit)
            up = up.clamp(min=-gemm1_limit, max=gemm1_limit)
            return (gate * torch.sigmoid(gate * gemm1_alpha) * (up + 1)).to(h.dtype)
        if gemm1_limit is not None:
            d = h.shape[-1] // 2
            gate = torch.nn.functional.silu(h[..., :d].float()).clamp(max=gemm1_limit)
            return (gate * h[..., d:].float().clamp(min=-gemm1_limit, max=gemm1_limit)).to(h.dtype)
        if swiglu_limit is not None:
            d = h.shape[-1] // 2
            return act_and_mul(torch.cat([h[..., :d].clamp(max=swiglu_limit),
                                          h[..., d:].clamp(min=-swiglu_limit, max=swiglu_limit)], dim=-1), "silu")
    else:
        assert gemm1_alpha is None and gemm1_limit is None and swiglu_limit is None
    if is_gated:
        return act_and_mul(h, activation)
    if activation == "silu":
        return torch.nn.functional.silu(h)
    if activation == "gelu":
        return torch.nn.functional.gelu(h)
    if activation == "relu2":
        return torch.square(torch.nn.functional.relu(h))
    raise ValueError(f"Unsupported activation: {activation=}, with {is_gated=}")


def fused_moe_block_fp8(x: torch.Tensor, w13_q: np.ndarray, w2_q: np.ndarray, w13_s: np.ndarray,
                        w2_s: np.ndarray, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                        block=(128, 128), routed_scaling_factor: float = 1.0, quant_form: str = "divide",
                        int8: bool = False, activation: str = "silu", is_gated: bool = True, **act_kw):
    """activation / is_gated / act_kw (gemm1_alpha, gemm1_limit, swiglu_limit): what stands between the two GEMMs (moe_activation); not gated, w13_q is [E, I, H].
    int8=True is the block-INT8 twin (torch_w8a8_block_int8_moe, test/registered/quant/test_block_int8.py:101-131):
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
        act = moe_activation(inter, activation, is_gated, **act_kw)
        aq, a_s, _ = group_quant(act, block[1], form=quant_form, dst=dst)
        o = mm(aq, w2_q[e], a_s, w2_s[e], block, return_fp32=True)
        y[sel] = (o * w_flat[sel].view(-1, 1)).to(x.dtype).to(torch.float32)
    out = (y.view(m, topk, hidden_out).sum(dim=1) * routed_scaling_factor).to(x.dtype)
    return out


def fused_moe_row_scaled(x: torch.Tensor, w13_q: np.ndarray, w2_q: np.ndarray, w13_s: np.ndarray, w2_s: np.ndarray,
                         topk_weights: torch.Tensor, topk_ids: torch.Tensor, int8: bool = False,
                         a1_scale: float = None, a2_scale: float = None, b1: torch.Tensor = None,
                         b2: torch.Tensor = None, routed_scaling_factor: float = 1.0,
                         apply_router_weight_on_input: bool = False, per_tensor_dynamic: bool = False,
                         activation: str = "silu", is_gated: bool = True):
    """The fused MoE with row scaling (block_shape None): per-token activation scales and per-channel weight scales
    (per_channel_quant; torch_w8a8_per_column_moe, test/registered/quant/test_int8_kernel.py:39-79, and its FP8 twin
    test/registered/moe/test_triton_moe_channel_fp8_kernel.py), or, FP8 with a1_scale / a2_scale given, one static
    activation scale per tensor and one weight scale per expert (fused_moe_triton_kernels.py:737-746,514-516;
    per_tensor_dynamic: that scale is max|A| / 448 of each GEMM's whole input instead).
    As in fused_moe_block_fp8 the routing weight multiplies the fp32 result of the GEMM it is attached to and the
    top-k sum runs in fp32 (fused_moe_triton_kernels.py:590-606,1084-1099).  Biases are added after the scales
    (:594-595).  w13_s [E, 2I] or [E]; w2_s [E, H] or [E]."""
    from .gemm import fp8_scaled_mm, int8_scaled_mm
    from .quant import dynamic_per_tensor_quant_fp8, per_token_quant_fp8, per_token_quant_int8, static_quant_fp8

    m, h = x.shape
    topk = topk_ids.shape[1]
    ids = topk_ids.reshape(-1).numpy()
    xa = x.view(m, 1, h).repeat(1, topk, 1).reshape(-1, h)
    mm = int8_scaled_mm if int8 else fp8_scaled_mm

    def quant(t, static):
        if int8:
            return per_token_quant_int8(t)
        if static is not None:
            return static_quant_fp8(t, static)
        if per_tensor_dynamic:
            q, s1 = dynamic_per_tensor_quant_fp8(t)
            return q, np.full((t.shape[0],), s1[0], dtype=np.float32)
        return per_token_quant_fp8(t)

    def wscale(sc, e, n):
        v = np.asarray(sc[e], dtype=np.float32).reshape(-1)
        return np.full((n,), v[0], dtype=np.float32) if v.size == 1 else v

    xq, xs = quant(xa, a1_scale)
    hidden_out = w2_q.shape[1]
    inter_dim = w13_q.shape[1] // 2 if is_gated else w13_q.shape[1]
    w_flat = topk_weights.reshape(-1).to(torch.float32)
    experts = [e for e in np.unique(ids) if e >= 0]
    # first GEMM + activation for every slot (slots of experts that live elsewhere stay zero, as the kernel writes
    # them), then one quantisation of the whole intermediate: a dynamic per-tensor scale spans all slots
    act_all = torch.zeros(m * topk, inter_dim, dtype=x.dtype)
    for e in experts:
        sel = np.nonzero(ids == e)[0]
        inter = mm(xq[sel], w13_q[e], xs[sel], wscale(w13_s, e, w13_q.shape[1]), bias=None if b1 is None else b1[e],
                   return_fp32=True)
        if apply_router_weight_on_input:
            inter = inter * w_flat[sel].view(-1, 1)
        act_all[sel] = moe_activation(inter.to(x.dtype), activation, is_gated)
    aq_all, as_all = quant(act_all, a2_scale)
    y = torch.zeros(m * topk, hidden_out, dtype=torch.float32)
    for e in experts:
        sel = np.nonzero(ids == e)[0]
        o = mm(aq_all[sel], w2_q[e], as_all[sel], wscale(w2_s, e, hidden_out), bias=None if b2 is None else b2[e],
               return_fp32=True)
        if not apply_router_weight_on_input:
            o = o * w_flat[sel].view(-1, 1)
        y[sel] = o.to(x.dtype).to(torch.float32)
    return (y.view(m, topk, hidden_out).sum(dim=1) * routed_scaling_factor).to(x.dtype)


# ---- expert-major ("grouped") MoE interface ------------------------------------------------------

def prepare_moe_input(topk_ids: np.ndarray, num_experts: int, n: int, k: int):
    """sgl-kernel/csrc/moe/prepare_moe_input.cu:12-93: per-expert row counts, their exclusive prefix (and the
    128-rounded one, :55-74), problem sizes (rows, 2n, k) / (rows, k, n), and the two permutations
    input_permutation[pos] = i // topk, output_permutation[i] = pos.  The reference places the members of one
    expert's span in the order its atomics land (:83-91); ascending flat index i is used here.  Ids outside
    [0, E) are skipped; their output_permutation entries are returned as -1 (unspecified in the reference).
    Returns (expert_offsets[E+1], blockscale_offsets[E+1], problem_sizes1[E,3], problem_sizes2[E,3],
    input_permutation[numel], output_permutation[numel])."""
    ids = np.asarray(topk_ids)
    topk = ids.shape[1] if ids.ndim == 2 else 1
    flat = ids.reshape(-1)
    counts = np.array([(flat == e).sum() for e in range(num_experts)], dtype=np.int32)
    offsets = np.zeros(num_experts + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts)
    bs_offsets = np.zeros(num_experts + 1, dtype=np.int32)
    bs_offsets[1:] = np.cumsum((counts + 127) // 128 * 128)
    ps1 = np.stack([counts, np.full_like(counts, 2 * n), np.full_like(counts, k)], axis=1).astype(np.int32)
    ps2 = np.stack([counts, np.full_like(counts, k), np.full_like(counts, n)], axis=1).astype(np.int32)
    in_perm = np.full(flat.size, -1, dtype=np.int32)
    out_perm = np.full(flat.size, -1, dtype=np.int32)
    fill = offsets[:-1].copy()
    for i, e in enumerate(flat):
        if 0 <= e < num_experts:
            in_perm[fill[e]] = i // topk
            out_perm[i] = fill[e]
            fill[e] += 1
    return offsets, bs_offsets, ps1, ps2, in_perm, out_perm


def shuffle_rows(x: np.ndarray, dst2src: np.ndarray) -> np.ndarray:
    """prepare_moe_input.cu:165-195: output row r = input row dst2src[r]."""
    return np.ascontiguousarray(x[np.asarray(dst2src, dtype=np.int64)])


def apply_shuffle_mul_sum(c: torch.Tensor, permutation: np.ndarray, factors: torch.Tensor, m: int) -> torch.Tensor:
    """prepare_moe_input.cu:248-298: out[i] = cast(sum_j f32(factors[i, j]) * f32(c[permutation[i*topk + j]])),
    fp32 accumulator, ascending j, each step one fused multiply-add as the compiled `sum += factor * val` is
    (the product of two 16-bit floats is exact in float64, so float64 multiply-add rounded to fp32 is that fma)."""
    topk = permutation.size // m
    rows = c[torch.from_numpy(np.asarray(permutation, dtype=np.int64))].to(torch.float64).view(m, topk, -1)
    acc = torch.zeros(m, c.shape[1], dtype=torch.float32)
    for j in range(topk):
        f = factors.reshape(m, topk)[:, j].to(torch.float64).view(m, 1) if factors is not None else 1.0
        acc = (f * rows[:, j] + acc.to(torch.float64)).to(torch.float32)
    return acc.to(c.dtype)


def fp8_blockwise_scaled_grouped_mm(aq: np.ndarray, a_s: np.ndarray, bq: np.ndarray, b_s: np.ndarray,
                                    problem_sizes: np.ndarray, expert_offsets: np.ndarray, out_dtype=torch.bfloat16):
    """One block-FP8 matmul per expert over its row span (test_fp8_blockwise_grouped_mm,
    sgl-kernel/tests/test_fp8_blockwise_moe.py:109-213: a_stack rows [offsets[g], offsets[g+1]) against b_stack[g]).
    aq [rows, K] codes, a_s [rows, K/128], bq [E, N, K] codes, b_s [E, N/128, K/128].  Rows in no span stay zero."""
    rows, n = aq.shape[0], bq.shape[1]
    out = torch.zeros(rows, n, dtype=out_dtype)
    for e in range(bq.shape[0]):
        m_e, lo = int(problem_sizes[e][0]), int(expert_offsets[e])
        if m_e > 0:
            out[lo:lo + m_e] = block_fp8_matmul(aq[lo:lo + m_e], bq[e], a_s[lo:lo + m_e], b_s[e], out_dtype=out_dtype)
    return out


def cutlass_fused_experts_fp8(x: torch.Tensor, w13_q: np.ndarray, w2_q: np.ndarray, w13_s: np.ndarray,
                              w2_s: np.ndarray, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                              quant_form: str = "reciprocal"):
    """The sequence of python/sglang/srt/layers/moe/cutlass_moe.py:185-341 on the functions above: quantise,
    gather to expert-major order, grouped GEMM 1, SiLU*mul, quantise, grouped GEMM 2, weighted top-k sum with
    the routing weights cast to the activation dtype first (:339).  Weights as [E, 2I, H] / [E, H, I] codes."""
    m, h = x.shape
    E, inter = w13_q.shape[0], w2_q.shape[2]
    offs, _, ps1, ps2, a_map, c_map = prepare_moe_input(topk_ids.numpy(), E, inter, h)
    xq, xs, _ = group_quant(x, 128, form=quant_form)
    rep_q, rep_s = shuffle_rows(xq, a_map), shuffle_rows(xs, a_map)
    c1 = fp8_blockwise_scaled_grouped_mm(rep_q, rep_s, w13_q, w13_s, ps1, offs[:-1], out_dtype=x.dtype)
    act = silu_and_mul(c1)
    aq, a_s, _ = group_quant(act, 128, form=quant_form)
    c2 = fp8_blockwise_scaled_grouped_mm(aq, a_s, w2_q, w2_s, ps2, offs[:-1], out_dtype=x.dtype)
    return apply_shuffle_mul_sum(c2, c_map, topk_weights.to(x.dtype), m)
