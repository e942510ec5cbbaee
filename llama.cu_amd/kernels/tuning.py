"""The numbers by which the dispatcher chooses between kernels that compute the same thing.

They were measured on one MI355X with the layer sizes of the Llama-3-8B shape (and checked on
the Llama-2-7B and Llama-3-70B shapes): they change which kernel runs and how it is launched,
never what comes out, so another shape or another card may want other numbers and nothing
else.  All of them are here, as data; ``ops`` and ``parts.linear`` read ``TUNING`` and hold
no such number of their own.  Replace fields (``dataclasses.replace``) or assign ``ops.TUNING``
to try others.
"""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class Tuning:
    # ---- the weight-streaming product for few rows (gemm_skinny.hip)
    skinny_rows: int = 16               # up to here it beats the library's product with a plain weight ...
    skinny_rows_packed: int = 24        # ... up to here with a packed weight, whose epilogues save the kernels around it
                                        # (whole decode steps: +9 % at 17 rows, +4 % at 24)
    skinny_rows_short_k: int = 24       # ... and up to here for packed weights with K <= skinny_short_k (q/k/v, output,
                                        # gate/up; it was 32 before the row-sharing product spread its tiles over all compute
                                        # units: now whole steps of 28 requests are 1 % faster and of 32 requests 2.7 % with 24)
    skinny_short_k: int = 8192
    skinny_rows_any_weight: int = 4     # so few rows always go to it
    skinny_small_weight: int = 1 << 24  # without a packed copy, beyond 4 rows only weights up to this many elements
    skinny_two_tiles_from: int = 6144   # packed: two tiles of 16 features a workgroup from this many features on ...
    skinny_four_tiles_from: int = 65536  # ... four for the widest, with more than 8 rows
    skinny_workgroups_per_cu: int = 4   # plain: as many tiles as still leave this many workgroups for each compute unit
    skinny_eight_waves_to: int = 8192   # eight waves share a workgroup's K up to this many output features, four beyond
    compute_units: int = 256            # of the card the numbers were measured on; ``for_device`` puts in the card's own
    # ---- the product that shares the rows through LDS (gemm_mid.hip, up to 256 rows)
    mid_long_k: int = 8192              # with a plain (not packed) weight only weights with a longer K than this (the down
                                        # projection) go to it at all; a packed weight with a longer K goes to it
    mid_long_k_rows: int = 11           # ... above this many rows (whole decode steps: 0.9 % faster at 12 rows, 3 % at 16;
                                        # 0.3 % slower at 11: below, the weight-streaming kernel with the norm in its epilogue)
    mid_swiglu_features: int = 8192     # gate/up with SwiGLU goes to it from this many rows of the weight on,
    mid_swiglu_rows: int = 14           # above this many rows of the batch (whole steps: 2.8 % at 16 rows, nothing at 14, slower below)
    mid_swiglu_max_rows: int = 192      # ... up to this many (at 160 and 192 rows 57 and 61 us against the library's 62 and 66 with
                                        # the activation kernel: whole steps 4 and 6 % faster; at 256 rows 78 against 73)
    mid_long_k_max_rows: int = 256      # the products cut over K go to it up to this many rows with a long K (the down
                                        # projection: 42 us against the library's 85 at 160 rows, 55 against 65 at 256)
    mid_short_k_max_rows: int = 192     # ... and up to this many with a shorter one (the output projection: 19 us against 25 to
                                        # 28 at 160 to 192 rows, no gain beyond)
    mid_qkv_rows: int = 16              # q/k/v with the rotation and the cache write in its epilogue goes to it above this
    mid_qkv_max_rows: int = 192         # many rows and up to this many, with a packed weight (whole decode steps over short
                                        # contexts: 1 to 2 % faster from 20 to 64 rows, 2.5 % at 80, 3.5 % at 128, 5 % at 144, even at 160
                                        # to 192; 1 to 2 % slower at 14 and 16 rows)
    mid_qkv_one_round_rows: int = 32    # ... beyond this many rows only if its workgroups (one for every 32 rows of the weight) are
                                        # no more than the compute units
    mid_add_norm_rows: int = 16         # a product with a short K that ends a branch (the output projection) goes to it with the residual
    mid_add_norm_max_rows: int = 32     # sum and the next norm's weight in its epilogue above this many rows and up to this many, while
                                        # its workgroups (one for 16 output features) run in one round: 11.9 us at 17 to 32 rows (the
                                        # weight-streaming kernel 13.1 to 16.9, planes and the norm kernel 14.2); whole steps 0.3 %
                                        # faster at 20 rows, 1.7 % at 32; 2 % slower at 16 and at 40 to 48, where the first product
                                        # of the feed-forward pays more for the rows' factors than the norm kernel cost
    mid_f32_rows: int = 32              # a product with 32-bit output (the output matrix, 1.05 GB) goes to it, uncut, above this many
    mid_f32_max_rows: int = 64          # rows and up to this many (whole steps 1.3 % faster at 40 rows, 1.9 % at 48, 0.7 % at 64;
                                        # nothing at 25 to 32)
    mid_min_slice_steps: int = 4        # a slice of K keeps at least this many macro-steps of 128
    mid_max_slices: int = 8
    # ---- the library's product of many rows (parts/linear.library_friendly_rows)
    library_rows: int = -1              # rows of zeros behind each half of a plain gate/up matrix: -1 times the library once per
                                        # shape at load and fills up where that is 15 % faster (the outcome can differ from box
                                        # to box near that mark); 0 never fills up; n > 0 fills each half up to a multiple of n
    # ---- the decode attention's cut of a request's keys into parts (attention_mfma.hip)
    decode_min_part_keys: int = 512     # no part shorter than this
    decode_max_parts: int = 32
    decode_few_workgroups: int = 128    # up to this many workgroups without parts: about one workgroup per compute unit
    decode_long_context: int = 2048     # between half the chip's worth of workgroups and all of it: parts only from here on
                                        # (rounded up to a power of two: from 1,025 keys),
    decode_long_part_keys: int = 1024   # of at least this many keys (with non-temporal loads of the keys, whole decode steps over
                                        # 2k keys: 5.5 % faster at 17 requests, 3.5 % at 20, 1.7 % at 22, nothing from 24 on),
    decode_long_max_parts: int = 4      # at most this many,
    decode_fill_slack: float = 0.07     # the fewest that fill whole waves of workgroups within this of the best


TUNING = Tuning()


def for_device(tuning: Tuning, device) -> Tuning:
    """``tuning`` with the facts of the card at ``device`` in the fields that are the card's (the number of compute
    units), not choices."""
    import dataclasses

    import torch
    units = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return tuning if units == tuning.compute_units or units <= 0 else dataclasses.replace(tuning, compute_units=units)
