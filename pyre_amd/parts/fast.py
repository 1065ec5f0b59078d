"""Choice of the faster kernels of the 16-bit path.

Each function returns None / False when its fast path does not take the case
(element type, sizes, alignment); the caller then runs the general kernel.
Nothing here changes what is computed, only by which kernel. Plain matrix
products with many rows go to the vendor's BLAS through ``torch.mm``, as the
reference's do (`pyre/model.py:84-87` are ``nn.Linear``); the true 32-bit path
never comes here.
"""

from __future__ import annotations

import torch

from pyre_amd.hip.ops import DEFAULT_UNITS, Partials

#: most rows the weight-streaming MFMA kernel takes; above, 16-bit products go to the kernel that keeps
#: up to 256 rows in a block where it pays and else to the BLAS library
SKINNY_MAX_ROWS = 64
#: the most partial sums of a weight-streaming product
SKINNY_MAX_KSPLIT = 12
#: up to this many rows the gate/up product and the SiLU-gate can be one weight-streaming kernel
#: (shapes whose features one round of the other kernel's blocks does not hold: the 32B shape's
#: at up to 24 rows)
FUSED_SILU_MAX_ROWS = 64
#: most rows of the kernel between the two, which keeps a step's rows against 64 rows of the weights
MID_MAX_ROWS = 256
MID_MAX_KSPLIT = 12
#: fewest rows at which that kernel takes the gate/up product with the SiLU-gate
MID_SILU_MIN_ROWS = 1
#: fewest rows at which its form with 128 rows of the weights a block takes a narrow product
#: (just above a size at which decode steps are captured, so that an eager step and its replay agree)
MID_WIDE_MIN_ROWS = 25


#: what the weight-streaming products reach while they stream, measured on the 7B shapes on an
#: MI355X, in bytes per microsecond over the whole chip; the time of one run of 128 k of a block
#: and of one more addend in the consumer, in microseconds
STREAM_BYTES_PER_US, STREAM_RUN_US, STREAM_PART_US = 6.5e6, 0.9, 0.1


def skinny_ksplit(m: int, n_out: int, k: int, units: int = DEFAULT_UNITS) -> int:
    """Into how many parts of k to split a weight-streaming product. A block (64 rows of the
    weights, 128 of wide ones) walks its part of k in dependent runs of 128, about 0.9 us
    each, and the blocks of a compute unit share its time: the product takes as long as the
    longest walk or as the unit with the most blocks needs for its bytes (6.5 TB/s over the
    ``units`` compute units), whichever is more; every part costs its consumer
    one more addend. The split with the least of that is chosen, at least four runs a part."""
    run_us, bytes_per_us, part_us = STREAM_RUN_US, STREAM_BYTES_PER_US, STREAM_PART_US
    tiles = -(-n_out // 16)
    row_blocks = -(-n_out // (128 if tiles >= 2048 else 64))
    runs = -(-k // 128)
    stream_us = 2.0 * n_out * k / bytes_per_us
    best, best_cost = 1, None
    for ks in range(1, SKINNY_MAX_KSPLIT + 1):
        per = -(-runs // ks)
        if ks > 1 and per < 4:
            break
        if -(-runs // per) != ks:
            continue  # would leave parts empty
        blocks = row_blocks * ks
        busiest = -(-blocks // units)
        cost = max(per * run_us, stream_us * busiest * units / blocks) + part_us * ks
        if best_cost is None or cost < best_cost - 1e-9:
            best, best_cost = ks, cost
    return best


def mid_ksplit(n_out: int, k: int, block_rows: int = 64, units: int = DEFAULT_UNITS) -> int:
    """Into how many parts of k the kernel that keeps a step's rows in a block (up to 256) splits a
    product, or 0 if it is not the one to take. A block has 64 rows of the weights; the kernel is at its best when the blocks
    of all parts fill the ``units`` compute units in one round, and beats the BLAS library where that
    takes at least two parts of 384 k or more (shorter parts gain nothing and cost the consumer
    another addend; measured on the 1.5B, 7B and 32B shapes: q/k/v, the
    attention output and the feed-forward's way down take 9 to 20 us where the library takes 19
    to 31, and 60 against 100 at 7B's way down; the wide gate/up product stays with the library)."""
    blocks = -(-n_out // block_rows)
    ks = min(units // blocks, k // 384, MID_MAX_KSPLIT)
    while ks > 1 and (ks - 1) * (-(-(-(-k // ks)) // 64) * 64) >= k:
        ks -= 1  # would leave a part empty
    return ks if ks >= 2 else 0


#: products whose library result is kept in float32 instead of being rounded to 16 bits:
#: q/k/v (rotated and rounded once afterwards) and the attention output projection (added
#: to the float32 residual). Measured on the tiny test models this halves the 16-bit
#: path's distance from an exact run; it costs about 2 % of a 2,048-token prefill.
LIBRARY_F32_ROLES = frozenset({"attn.qkv", "attn.out"})


def _is_bf16(ctx, lin, x) -> bool:
    return (ctx.runtime.dtype == torch.bfloat16 and lin.weight.dtype == torch.bfloat16
            and x.dtype == torch.bfloat16)


def narrow_kernel(n: int, n_out: int, k: int, options: dict | None = None,
                  units: int = DEFAULT_UNITS) -> tuple[str, int, bool]:
    """Which of our kernels takes a 16-bit product of ``n`` rows whose result is handed on as partial
    sums: ("stream", parts of k, False) for the weight-streaming kernel, ("block", parts, wide) for the
    kernel that keeps the step's rows in a block (``wide``: 128 rows of the weights a block instead
    of 64), ("", 0, False) for neither (the BLAS library then). A function of the sizes (and of the
    device's compute units, which an engine reads once) alone; the
    thresholds in rows lie just above sizes at which decode steps are captured, so that an eager step
    and its replay at the padded size agree."""
    opt = options or {}
    block = opt.get("mid_gemm", True)
    if block and opt.get("mid_wide_min_rows", MID_WIDE_MIN_ROWS) <= n <= MID_MAX_ROWS:
        # With 128 rows of the weights a block, where such blocks fill three quarters of the chip at
        # least: a block's bytes are the step's rows of X and its rows of W, over its part of k, and
        # with as many of the one as of the other they are fewest (at few rows of X a stage, and the
        # barrier that goes with it, carries twice the bytes). From 25 rows on the weight-streaming
        # kernel slows down (64 activations come from L2 once per 128 rows of weights, and four
        # times the LDS reads and MFMAs sit between a run's arrival and the next run's request),
        # this one does not. Measured in steps of the 7B shape against the weight-streaming kernel:
        # 4.43 against 4.47 ms at 32 requests, 5.20 against 5.29 at 48, 5.74 against 5.88 at 64 (at 8
        # and 16: 3.46 against 3.44, 3.79 against 3.77); of the 32B shape 35.5 against 36.2 at 64.
        # Against 64 rows of the weights a block: 7.78 against 7.94 ms at 96 requests, 8.86 against
        # 8.90 at 128, 12.56 against 12.63 at 192, 15.25 against 15.34 at 256.
        ks = mid_ksplit(n_out, k, 128, units)
        if ks and 4 * -(-n_out // 128) * ks >= 3 * units:
            return "block", ks, True
    if n <= SKINNY_MAX_ROWS and opt.get("skinny_gemm", True):
        ks = skinny_ksplit(n, n_out, k, units)
        if block and opt.get("mid_small", True) and -(-n_out // 64) * ks < units and mid_ksplit(n_out, k, 64, units):
            # A product so small that the weight-streaming kernel's blocks do not fill the compute
            # units (the 1.5B shape's: 96, 72 and 240 blocks) is latency all the way, and the other
            # kernel, whose loads go straight into a ring in LDS, starts sooner: 1.7 % of a step of
            # 8 requests of that shape, 3 % at 32, 4 % at 64. Where the blocks fill the chip (7B:
            # 504) it is 3 % slower at 8 rows.
            return "block", mid_ksplit(n_out, k, 64, units), False
        return "stream", ks, False
    if n <= MID_MAX_ROWS and block:
        ks = mid_ksplit(n_out, k, 64, units)
        if not ks and int(block) == 2:  # tests: also where it does not pay, as with a tiny model
            ks = 2 if k > 64 else 1
        if ks:
            return "block", ks, False
    return "", 0, False


def linear(lin, ctx, x, n, out):
    from pyre_amd.hip import ops

    rt = ctx.runtime
    if not _is_bf16(ctx, lin, x):
        return None
    k, n_out = lin.in_features, lin.out_features
    streams = rt.options.get("skinny_gemm", True) and ops.gemm_skinny_supports(
        min(n, SKINNY_MAX_ROWS), n_out, k, x.stride(0), lin.weight.stride(0))
    library = rt.options.get("library_gemm", True)
    if out is not None:
        # float32 results wanted in place (the head's logits)
        if streams and (n <= SKINNY_MAX_ROWS or not library):  # no split, 64 rows at a time
            for r0 in range(0, n, SKINNY_MAX_ROWS):
                rows = min(SKINNY_MAX_ROWS, n - r0)
                ops.gemm_skinny_bf16(x[r0:r0 + rows], lin.weight, out[r0:r0 + rows], rows, 1)
        elif library:  # many rows (a large decode step, or every row of a portion): one pass over the weights
            torch.mm(x if n == x.shape[0] else x[:n], lin.weight.t(), out_dtype=torch.float32, out=out)
        else:
            return None
        return Partials(out.view(1, n, n_out), lin.bias)
    kernel, ks, wide = narrow_kernel(n, n_out, k, rt.options, rt.compute_units)
    if kernel == "stream" and not streams:
        kernel = ""
    if kernel == "block" and not ops.gemm_mid_supports(n, n_out, k, x.stride(0), lin.weight.stride(0)):
        kernel, ks = ("stream", skinny_ksplit(n, n_out, k, rt.compute_units)) if streams and n <= SKINNY_MAX_ROWS else ("", 0)
    if kernel:
        buf = ctx.workspace.get(f"linear.{lin.role}.partials", (ks, n, n_out), torch.float32)
        if kernel == "stream":
            ops.gemm_skinny_bf16(x, lin.weight, buf, n, ks)
        else:
            ops.gemm_mid_bf16(x, lin.weight, buf, n, ks, wide=wide)
        return Partials(buf, lin.bias)
    if not library:
        return None
    if lin.role in rt.options.get("library_f32_roles", LIBRARY_F32_ROLES):
        buf = ctx.workspace.get(f"linear32.{lin.role}", (n, n_out), torch.float32)
        torch.mm(x if n == x.shape[0] else x[:n], lin.weight.t(), out_dtype=torch.float32, out=buf)
    else:
        buf = ctx.workspace.get(f"linear16.{lin.role}", (n, n_out), torch.bfloat16)
        torch.mm(x if n == x.shape[0] else x[:n], lin.weight.t(), out=buf)
    return Partials(buf.view(1, n, n_out), lin.bias)


def gate_up_silu(lin, ctx, x, n, act) -> bool:
    """silu(x gate^T) * (x up^T) in one kernel: the kernel that keeps all rows in a block for up to
    256 rows where one round of blocks holds the features, else the weight-streaming kernel for a
    decode step's few rows."""
    from pyre_amd.hip import ops

    if not _is_bf16(ctx, lin, x) or lin.bias is not None:
        return False
    if ctx.runtime.options.get("mid_silu_min_rows", MID_SILU_MIN_ROWS) <= n <= MID_MAX_ROWS:
        # blocks of 64 features (96 where that is what it takes, up to 128 rows) against all rows,
        # where one round of blocks holds them. Measured on the 1.5B shape: 17 us against the
        # library's product and the SiLU-gate kernel's 29 at 65 to 128 rows, 26 against 30 at 192, 28 at 256;
        # on the 7B shape 55 against 66 at 128, and at 256 rows, as on the 32B shape, two rounds of
        # blocks: those stay with the library. With blocks of 32 and 64 rows of X for steps that
        # small it is ahead of the weight-streaming kernel at every size: on the 7B shape 3.20
        # against 3.23 ms a step at one request, 3.44 against 3.49 at 8, 3.77 against 3.87 at 16,
        # 4.46 against 4.56 at 32, 5.87 against 6.13 at 64; on the 1.5B shape by 1 to 4 %.
        mid = ctx.runtime.options.get("mid_gemm", True)
        fits = mid and ops.gemm_mid_supports(n, lin.out_features, lin.in_features, x.stride(0), lin.weight.stride(0))
        if fits and (ops.gemm_mid_silu_blocks(n, lin.out_features) <= ctx.runtime.compute_units or int(mid) == 2):
            ops.gemm_mid_silu_bf16(x, lin.weight, act, n)
            return True
    if n > FUSED_SILU_MAX_ROWS or not ctx.runtime.options.get("skinny_gemm", True):
        return False
    if not ops.gemm_skinny_supports(n, lin.out_features, lin.in_features, x.stride(0), lin.weight.stride(0)):
        return False
    ops.gemm_skinny_silu_bf16(x, lin.weight, act, n)
    return True


#: rows of the prompt-portion kernel's work list that one launch takes (the grid's second dimension)
PREFILL_MAX_LAUNCH = 65535


def rope_in_attention(mixer, ctx, qkv, cache, rotary_dim: int) -> bool:
    """Whether the step's attention kernel can finish the q/k/v product itself (sum of the partial
    sums, bias, rotation, the cache write): a step of single tokens only, on the 16-bit path's decode
    kernel, full-head rotation, heads of up to 128 elements. The kernel between product and attention
    is then left out; the bits are the same. A function of the step's shape and the model's sizes."""
    from pyre_amd.hip import ops

    s = mixer.spec
    hb = ctx.host
    if ctx.dtype != torch.bfloat16 or cache["k"].dtype != torch.bfloat16 or qkv.data.dtype != torch.float32:
        return False
    if not ctx.runtime.options.get("mfma_attention", True) or not ctx.runtime.options.get("rope_in_attention", True):
        return False
    if rotary_dim != s.head_dim or len(hb.arrays["attention.prefill_tiles"]) or \
            len(hb.arrays["attention.decode_tokens"]) != ctx.n_tokens:
        return False
    return ops.attn_decode_work_rope_supports(s.head_dim, cache.page_size, s.num_heads, s.num_kv_heads, qkv.stride)


def attention(mixer, ctx, q, o, cache, rope=None) -> bool:
    """``rope``: (the q/k/v product's partial sums, cos, sin) when :func:`rope_in_attention` said that
    the decode kernel finishes the product; ``q`` is then not read."""
    from pyre_amd.hip import ops
    from pyre_amd.parts.attention_work import (decode_alone, decode_capacity, decode_items, prefill_items,
                                                prefill_slots)

    s = mixer.spec
    k_pages, v_pages = cache["k"], cache["v"]
    if ctx.dtype != torch.bfloat16 or k_pages.dtype != torch.bfloat16:
        return False
    if not ctx.runtime.options.get("mfma_attention", True):
        return False
    if not ops.attn_mfma_supports(s.head_dim, cache.page_size, s.num_heads, s.num_kv_heads):
        return False
    hb = ctx.host
    dec, tiles = hb.arrays["attention.decode_tokens"], hb.arrays["attention.prefill_tiles"]
    n_dec, n_tiles = len(dec), len(tiles)
    if n_dec:
        # The launch's size follows from the step's rounded sizes and the list from the rounded
        # number of requests, so that a step gives bit for bit the same result whether it runs
        # eagerly or as a replayed graph at those sizes.
        rows, _ = hb.decode_shape()
        units = mixer.units
        capacity = decode_capacity(rows, s.num_heads, s.num_kv_heads, units)
        listed_blocks = int(hb.arrays[mixer.decode_work_name].reshape(-1)[0])
        if listed_blocks > capacity:  # the kernel would leave the rest of the list undone, silently
            raise RuntimeError(f"the decode attention's work list has {listed_blocks} blocks, its launch {capacity}")
        items = decode_items(s.num_heads, s.num_kv_heads)
        acc = ctx.workspace.get("attn.part_acc", (capacity, items, 16, s.head_dim), torch.float32)
        ml = ctx.workspace.get("attn.part_ml", (capacity, items, 16, 2), torch.float32)
        counters = ctx.workspace.get("attn.counters", (capacity, items), torch.int32, zeroed=True)
        alone = decode_alone(rows, s.num_heads, s.num_kv_heads, units)
        if rope is not None:
            qkv, cos, sin = rope
            ops.attn_decode_work_rope_bf16(qkv, cos, sin, cache.slots, o, k_pages, v_pages, cache.writes,
                                           ctx.arrays[mixer.decode_work_name], capacity, ctx.positions,
                                           ctx.seq_of_token, cache.table, acc, ml, counters, alone, s.num_heads,
                                           s.num_kv_heads, s.head_dim, cache.page_size, mixer.scale, cache.window)
        else:
            ops.attn_decode_work_bf16(q, o, k_pages, v_pages, ctx.arrays[mixer.decode_work_name], capacity,
                                      ctx.positions, ctx.seq_of_token, cache.table, acc, ml, counters, alone,
                                      s.num_heads, s.num_kv_heads, s.head_dim, cache.page_size, mixer.scale,
                                      cache.window)
    if n_tiles and s.head_dim <= 128:
        work = hb.arrays[mixer.prefill_work_name]
        n_slots = prefill_slots(work)
        if 8 * len(work) > ctx.arrays[mixer.prefill_work_name].numel():
            raise RuntimeError(f"the prompt attention's work list has {len(work)} blocks, its step array holds "
                               f"{ctx.arrays[mixer.prefill_work_name].numel() // 8}")
        per_slot = prefill_items(s.num_heads, s.num_kv_heads) * ops.attn_prefill_waves(s.num_heads, s.num_kv_heads)
        partials = counters = None
        if n_slots:
            partials = ctx.workspace.get("attn.prefill_partials", (n_slots, per_slot, s.head_dim // 32 * 1024 + 128),
                                         torch.float32)
            counters = ctx.workspace.get("attn.prefill_counters", (n_slots, per_slot), torch.int32, zeroed=True)
        listed = ctx.arrays[mixer.prefill_work_name]
        for at in range(0, len(work), PREFILL_MAX_LAUNCH):  # a launch takes 65,535 rows of the list
            count = min(PREFILL_MAX_LAUNCH, len(work) - at)
            ops.attn_prefill_work_bf16(q, o, k_pages, v_pages, listed[8 * at:], count, partials, counters, n_slots,
                                       ctx.positions, ctx.seq_of_token, cache.table, s.num_heads, s.num_kv_heads,
                                       s.head_dim, cache.page_size, mixer.scale, cache.window)
    elif n_tiles:
        ops.attn_prefill_bf16(q, o, k_pages, v_pages, ctx.arrays["attention.prefill_tiles"], n_tiles, ctx.positions,
                              ctx.seq_of_token, cache.table, s.num_heads, s.num_kv_heads, s.head_dim,
                              cache.page_size, mixer.scale, cache.window)
    return True
