"""What the dispatching operations may choose, and the sizes at which launch plans change their
shape: one object per model runner, handed to the operations through the step.

Nothing here changes what is computed, only which kernel computes it and how its work is cut.
Tests and measurements make an object with other values for an engine of their own; two engines in
one process do not share it, and a recorded decode step is kept under the values it was recorded
with."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class KernelChoices:
    # the matrix-instruction kernels where operand types and sizes fit them; off: every product /
    # every attention goes through the plain-precision kernels (the 32-bit model's always do)
    fast_gemm: bool = True
    fast_attention: bool = True
    # products of a few rows more than a multiple of 1,024 (at most tail_rows_most): those rows in a launch of
    # their own (ops.mfma.tail_rows)
    tail_rows_apart: bool = True
    tail_rows_most: int = 64
    # decoding, up to 16 tokens whose keys are cut into splits: the splits' join inside the output projection
    join_project: bool = True
    # decoding, 17 to 64 tokens with the keys in one split: rotation and cache write inside the attention kernel
    decode_rope: bool = True
    # decoding with heads of 64, the most tokens whose q/k/v product is still cut over k and added into a cleared
    # buffer, so that the attention kernel rotates and writes the cache (without decode_rope: 64, as for every
    # other step). Measured at the 1B sizes and a context of 2,048, ms a step with 64 / 128 here: 65 tokens
    # 2.125 / 2.044, 80: 2.287 / 2.218, 96: 2.504 / 2.473, 112: 2.916 / 2.898; 128: 3.216 / 3.287 on one box and
    # 3.268 / 3.195 on another; 160 tokens with 64 / 256: 3.630 / 3.697, 256: 5.069 / 5.236.
    qkv_sum_rows_decoding: int = 96
    # The same with heads of 128 (the rotation kernel behind the product, not the attention kernel). Measured at a
    # context of 2,048 over 8 layers, ms a step with 64 / 96 / 128 here: 3B sizes 65 tokens 1.921 / 1.840 / 1.847, 96:
    # 2.151 / 2.053 / 2.057, 112: 2.432 / 2.403 / 2.340, 128: 2.564 / 2.556 / 2.498; 8B sizes 65: 2.313 / 2.223 / 2.218,
    # 96: 2.568 / 2.466 / 2.467, 112: 2.879 / 2.864 / 2.806, 128: 3.014 / 3.030 / 2.984.
    qkv_sum_rows_decoding_128: int = 128
    # prompt attention: work items of half the rows where a step has few items
    prefill_half_rows: bool = True
    # Workgroups (of four wavefronts) the decode kernel should have at most when it cuts the keys: one
    # per compute unit (None: the device is asked for their number). Measured on the 256 compute units
    # of an MI355X at batch 8 and a context of 4,096: 0.948 ms a step with 256, 0.969 with 512, 0.998
    # with 1,024, 1.036 with 128; with 384 (one and a half per compute unit) 1.000.
    decode_blocks_wanted: int | None = None
    # Decoding with more workgroups than half the compute units (from 17 requests on with 8 kv heads), where one
    # per compute unit leaves the keys whole: the keys are cut where the host runtime's estimate says so
    # (ops.mfma.decode_cut, csrc/host/decode_plan.cpp). Measured at the 1B sizes (ms a step, keys whole / cut),
    # requests of one length: a context of 8,192: 17 requests 2.061 / 1.840 (5 splits), 20: 2.103 / 1.954 (3),
    # 24: 2.129 / 2.088 (4), 28 and 32: whole is best, 33: 3.170 / 2.618 (6), 40: 3.384 / 2.889 (4), 48: 3.681 /
    # 3.179 (2), 56 and 64: whole, 72: 5.071 / 4.664 (3); a context of 2,048: whole is best or equal everywhere
    # (17 requests 1.186 / 1.218, 33: 1.511 / 1.496); 16,384: 17 requests 3.171 / 2.556, 33: 5.440 / 4.049.
    # The same estimate judges one or two splits more where one workgroup per compute unit takes 2 to 6 splits
    # (5 to 16 requests): requests of one length keep that plan, requests of different lengths gain (12 requests
    # of 1,024 to 16,384 tokens 1.539 / 1.336, 11: 1.882 / 1.582).
    decode_cut_most: int = 8            # splits at most where the keys would be whole (1: the estimate is not asked)
    decode_cut_tbs: float = 6.0         # TB/s the keys stream at where the compute units share them evenly
    decode_cut_key_ns: float = 9.5      # ns a compute unit needs per key of a head of 64 that it is given
    decode_cut_lone_ns: float = 8.3     # the same for a unit's only piece where others hold two (it ends on a draining chip)
    decode_cut_piece_us: float = 0.5    # and per piece
    decode_cut_join_us: float = 4.6     # a cut costs the join kernel (17 requests and more)
    decode_cut_rope_us: float = 4.8     # and the rotation kernel, where the single split would have rotated itself
    decode_cut_each_us: float = 1.0     # and this per split
    decode_cut_gain: float = 0.05       # and must promise this fraction of the whole keys' time
    # Portions of prompts: work items (a span of rows x a group of heads) the prefill kernel should
    # have at least (None: two per compute unit, three where the step has more than half a compute unit's
    # number already); with prefill_cut_items or fewer (None: three quarters of the compute units' number;
    # measured: 256 items cut in two were 3 % slower than whole, and 224 to 256 items cut in three or four
    # no faster even behind 32,768 tokens), the longest item's keys are cut into that many runs of at least
    # prefill_min_run keys, and the others' into runs of the same length.
    prefill_items_wanted: int | None = None
    prefill_cut_items: int | None = None
    prefill_min_run: int = 512
    prefill_max_splits: int = 16
    # Two runs are not worth their join: a 256-token portion beside 17 decoded tokens at the 1B sizes takes
    # 2.18 ms in two runs against 2.07 whole behind 1,024 tokens, 2.28 against 2.27 behind 2,048 (four
    # runs: 2.20), and behind 3,000 tokens 2.32 in three or six runs against 2.49 whole.
    # (A whole prompt of 2,048 tokens, whose last rows' items walk twice the average, was also tried with
    # the items behind 1,024 keys cut in two: 6.5 to 6.6 ms against 5.95 whole; the partial outputs and
    # the join cost more than the evener load wins.)
    prefill_min_splits: int = 3
    # More than a quarter of a workgroup per compute unit (65 to 128 items on 256 units: portions of 257
    # to 512 tokens of 32 heads): the keys are cut only where an item has at least this many keys for
    # every item of the step, since whole keys in items of half the rows are faster until then and the
    # join costs 13 us a layer whatever the length. Measured at the 1B sizes beside 17 decoded tokens (ms a
    # step, cut / whole): 320 tokens behind 2,048: 2.55 / 2.32, behind 4,096: 2.61 / 2.63, behind 8,192:
    # 2.91 / 3.29; 512 tokens behind 1,024: 2.83 / 2.49, behind 4,096: 3.10 / 2.95, behind 8,192: 3.55 / 3.62,
    # behind 16,384: 4.44 / 4.97; 768 tokens (192 items, cut in four) behind 8,192: 4.85 / 4.85, behind 16,384:
    # 6.31 / 6.85, behind 32,768: 9.12 / 10.91. (Up to 64 items the cut never lost: 256 tokens behind 8,192:
    # 2.53 / 3.09.)
    # For heads of 64; a key of a head of 128 is twice the work, and half as many keys are long: at the 8B
    # sizes (8 layers) 768 tokens behind 8,192: 5.46 / 6.32, at the 3B sizes 3.53 / 4.68, behind 1,024 whole
    # keys win at both (4.33 / 4.42 and 2.64 / 2.73 whole / cut).
    prefill_cut_keys_per_item: int = 64

    def key(self) -> tuple:
        return tuple(self.__dict__.values())


# What an operation uses when it is called without a step (a kernel on its own).
DEFAULT = KernelChoices()


def choices_of(step) -> KernelChoices:
    return getattr(step, "choices", None) or DEFAULT
