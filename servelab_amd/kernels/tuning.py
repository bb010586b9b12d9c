"""The numbers that choose between kernels, in one place.

Kernel *limits* (how many rows a kernel can take, which head sizes) stay with
the kernels' wrappers in the kernel table (``*_ops.py``): they are facts of the code.  What is here
are *choices* that were measured on one MI355X with the projection sizes of the
Qwen2.5 7B, 32B and 72B shapes; another GPU or another architecture's sizes may
want others.  ``HipOps(dtype, device, tuning=Tuning(wide_min_m=...))`` takes a
changed set; every field becomes an attribute of the kernel table under its
upper-case name (``ops.WIDE_MIN_M``), which is what the routing code reads.
"""
from dataclasses import dataclass, fields


@dataclass
class Tuning:
    # ---- weight layouts
    # both copies of a matrix (row-major for the library, tiled for the few-rows kernels) are kept
    # while they stay below this share of the device's memory; beyond it only the tiled copy
    dual_memory_share: float = 0.45
    # a model beyond that keeps the tiled copy of every matrix and, while all copies stay below this
    # share of the device's memory, the row-major copy of as many matrices as fit as well, in the order
    # they are loaded: their products of many rows go straight to the library (72B shape, 145 GB of
    # weights: 77 GB of row-major copies, 44 of 80 layers; writing a matrix row-major into the scratch
    # buffer before each of its products was a fifth of a 2,048-token prefill)
    rows_copies_memory_share: float = 0.72
    # the matrices whose few-rows products add to the residual stream get a further copy in tiles of fewer
    # than 16 rows where those go round the CUs more evenly (HipOps.producer_tile_height), while all copies
    # stay below this share of the device's memory and the busiest CU pulls at least min_gain less (32B shape,
    # 5120 columns, 512 tiles of 10 rows for 320 of 16: a quarter less, +6 % tokens/s at batch 8, +2 % at batch 1;
    # 7B shape, 3584 columns, 256 tiles of 14 for 224 of 16: a twelfth less and nothing gained end to end)
    lower_tiles_memory_share: float = 0.55
    lower_tiles_min_gain: float = 0.15

    # few-rows products of at most 8 rows load x for two k-steps at once (gemm.hip, stream_k2)
    pair_x_loads: bool = True
    # Up to how many rows a step takes the few-rows kernels with the residual add, the norm and the
    # rotation fused in (16 at most: the rows of one matrix instruction), by the width of the residual
    # stream: (width up to which, rows) pairs.  Those kernels read all rows of x again for every tile of 16
    # rows of W, the LDS-staged ones once for 128 or 256, at the price of three more kernels a layer; the
    # wider the stream, the fewer rows the fused ones are ahead for (ms a decode step, contexts of 4,096,
    # fused up to 16 / 8 / 0 rows: 7B shape, width 3,584, 8 requests 3.14 / 3.14 / 3.59, 16 requests 3.64 / 3.97
    # / 3.99; 32B shape, 5,120: 8 requests 12.6 / 12.5 / 13.2, 16 requests 14.9 / 14.8 / 14.7; 72B shape, 8,192,
    # whose gate/up has no form that keeps x in registers: 1 request 25.2 / 25.2 / 24.2, 8 requests 26.3 / 26.3 /
    # 25.6, 16 requests 31.1 / 27.3 / 27.3)
    fused_norm_max_m: int = 16
    fused_rows_by_width: tuple = ((4096, 16), (6144, 8), (1 << 30, 0))

    # ---- products of 17 and more rows over the tiled copy
    # from this many rows on two tiles of W share one read of x (gemm_wide / gemm_mid)
    wide_min_m: int = 17
    # the LDS-staged kernel splits K until about this many workgroups stream W
    # (fewer splits, fewer partial sums); 224 of 256 CUs busy measured best for o and down
    mid_target_workgroups: int = 224
    # the same when the next norm adds the partial sums of a residual delta
    mid_deferred_workgroups: int = 224
    # fewer splits when the reader adds the partial sums itself (their bytes count twice)
    mid_partial_workgroups: int = 128
    # workgroups of 8 wavefronts (16 tiles of W per pass over x) if this many remain, else 4
    mid_wide_workgroups: int = 128
    # matrices of this many elements take the LDS-staged kernel at 17..32 rows ...
    mid_min_elements: int = 1 << 19
    # ... and of this many at 33..128 rows (smaller ones: two tiles a workgroup straight from L2, up to 64 rows).
    # Both were 48 M and 8 M elements while the kernel had workgroups of four wavefronts only; as it is, it
    # wins at every size measured: decode steps of 24 / 32 requests, 7B shape (the output projection, 12.8 M
    # elements) 4.33 -> 4.23 / 4.65 -> 4.54 ms, 32B shape 16.3 -> 16.0 / 17.7 -> 17.2 ms; the 0.5B shape (matrices
    # of 0.8 to 8.7 M elements) at 24 / 48 / 80 / 128 requests 1.58 -> 1.32 / 2.05 -> 1.61 / 5.46 -> 1.75 / 5.11 ->
    # 2.12 ms (beyond 64 rows its products went to the library, outside the captured step), 1.5B at 48 /
    # 128: 2.83 -> 2.70 / 5.21 -> 3.59 ms, 3B at 48 / 128: 4.16 -> 4.02 / 6.24 -> 5.35 ms
    mid_min_elements_many: int = 1 << 19
    # matrices of fewer elements than this stay off the block kernel (tiles of 256 rows of x) at 129 rows and more
    block_min_elements: int = 8 << 20

    # ---- the wavefront-per-column products (float32 table, bfloat16 fallbacks)
    # up to 16 rows of x go through LDS once per 32 columns of W instead of through L1 once per 4
    rows_through_lds: bool = True

    # ---- products over the row-major copy in tiles of 256 rows of x by 128 rows of W (gemm_block)
    # matrices of at most block_max_n rows (q/k/v, o, down: K is split over workgroups until every CU has
    # one; gate/up and the head have tiles enough for the library) take it from block_min_m rows of x
    # on, where the LDS-staged kernel ends, up to block_max_m (7B shape, against the library's tuned
    # kernels at 160 / 256 / 512 rows: down 44 / 46 / 83 us against 62 / 65 / 109, o 15 / 17 / 23 against 34 /
    # 32 / 31, q/k/v 20 / 22 / 35 against 31 / 38 / 37; a third tile of 256 rows makes it read W a third time
    # and the library wins: 544 rows down 124 against 114 us).  Below block_min_m it was measured too:
    # alone faster than the LDS-staged kernel (down at 64 / 128 rows 27 / 33 against 38 / 62 us), inside a
    # decode step of 24 to 128 requests 2-5 % slower, so those rows stay where they were.
    block_max_n: int = 8192
    block_min_m: int = 129
    block_max_m: int = 512
    # matrices with rows of this many values and more (the down projection) take tiles of 256 x 256 from
    # 257 rows of x up to this many (7B shape, down at 768 / 1,024 / 1,536 rows: 83 / 111 / 168 us)
    block_square_min_k: int = 8192
    block_square_max_m: int = 1536

    # ---- few-rows consumer products on workgroups that stay
    # tiles per CU from which walking the tiles beats a workgroup per tile (gate/up: 9, head: 37;
    # q/k/v with one or two tiles a CU has nothing to walk)
    resident_min_rounds: int = 3

    # ---- library products
    # products of fewer than library_padded_max_m rows run on a multiple of library_row_step rows:
    # few distinct shapes, each of which the start-up tuning can time
    library_row_step: int = 32
    library_padded_max_m: int = 512

    # ---- attention
    # wavefronts a decode launch of the general (float32) kernel aims for when it splits the context
    general_attention_waves: int = 4096
    # single tokens of no more (request, kv head) pairs than CUs, a wavefront per share of a pair's keys:
    # the estimate of a launch's time that picks the number of shares (HipOps._decode_shares): a trip
    # to memory of a wavefront (two key blocks), the rate at which a CU streams keys and values, a
    # wavefront more on every CU, and a batch of sixteen partial results in the combine kernel
    few_trip_us: float = 1.675
    few_stream_gbs_per_cu: float = 28.05
    few_wave_us: float = 0.922
    few_batch_us: float = 0.463
    # single tokens, no more (request, kv head) pairs than CUs: a workgroup of eight wavefronts takes a pair's keys
    # and merges in LDS (no partial results in memory, no second kernel) once there are group_attention_fill
    # times the share of group_attention_from pairs a CU, by the length of the longest context in key blocks;
    # below, a wavefront takes a share and the combine kernel merges.  Merged, a pair's keys come through one
    # CU, so it pays where contexts are short or nearly every CU has a pair.  7B and 32B shapes, us a layer,
    # merged against the best number of shares: contexts of 512, 112 / 144 / 256 pairs: 10.9 / 11.3 / 13.4
    # against 11.2 / 12.8 / 16.3; of 1,024, 128 / 192 / 224 pairs: 18.4 / 22.4 / 23.1 against 16.0 / 21.7 / 25.9;
    # of 2,048, 192 / 224 / 256 pairs: 41.4 / 42.9 / 45.8 against 37.4 / 45.3 / 47.7; of 4,096, 224 / 240 / 256
    # pairs: 83.1 / 85.6 / 89.4 against 81.8 / 87.1 / 89.4; of 8,192 and 16,384, 256 pairs: 175 and 345 against
    # 168 and 329 (a share above 1: never).  Contexts of up to 256 keys merge from one pair on (1 to 24
    # requests at 128 / 192 / 256 keys: 4.6-4.9 / 5.1-6.0 / 5.6-7.2 against 5.1-6.0 / 6.6-8.3 / 6.5-8.1 us; at 384 keys
    # both forms take the same time, from 512 on shares win: 8 requests 7.1 against 10.0 us).  Whole decode steps of the 7B shape: 32 requests at 1,024 keys
    # 3.92 -> 3.84 ms (in shares), 60 at 2,048 keys 4.98 -> 4.81 ms (merged); 48 at 1,024 keys 3.95 ms merged, 4.03 in shares.
    group_attention_fill: float = 1.0
    group_attention_from: tuple = ((8, 1 / 1024), (16, 0.45), (32, 0.7), (64, 0.85), (128, 0.97), (1 << 30, 1.01))
    # With more pairs than CUs the form is taken by an estimate of the launch's time, whose constants
    # are fitted to 63 launches of 288 to 1,024 pairs over contexts of 640 to 4,096 (3.5 % rms; the form
    # taken is 0.8 % slower than the best measured one on average, 6 % at worst).  The keys and values
    # stream at many_stream_gbs_per_cu GB/s times the CUs (6.3 TB/s on 256).  Wavefronts that take a
    # share each are spread over the CUs, and the launch takes as long as if every CU had as many as
    # the fullest (a factor of ceil(w / CUs) CUs / w; with more than many_crowded_waves a CU only
    # many_crowded of what it exceeds 1 by), no less than a wavefront's trips to memory, many_trip_us
    # for two key blocks, plus many_share_us per share and many_combine_us for the second kernel.
    # The workgroups that merge in LDS pay many_merged_rounds of that factor (those of the last round
    # have the chip to themselves) and many_merged_base overall.  Of estimates within many_fewer_within
    # of the lowest, the form with the fewest shares is taken.  Contexts of 4,096, us a layer for 72 / 104
    # / 112 / 144 / 160 requests of 4 kv heads: 110 / 153 / 160 / 207 / 228 (in 4 / 3 / 4 / 3 / 2 shares),
    # against 126 / 206 / 208 / 256 / 264 when more pairs than CUs meant two shares up to 384 pairs,
    # then one, or merged where the rounds were nearly full.
    many_stream_gbs_per_cu: float = 24.6
    many_trip_us: float = 2.95
    many_share_us: float = 0.84
    many_combine_us: float = 2.05
    many_crowded_waves: int = 3
    many_crowded: float = 0.46
    many_merged_rounds: float = 0.57
    many_merged_base: float = 1.048
    many_fewer_within: float = 1.02
    # Two launches instead: the sequences that fill whole rounds of the CUs merged in the workgroup,
    # which then runs at the rate of the stream, and the others as a launch of few pairs, which costs
    # its own stream or its wavefronts' trips and many_second_launch_us on top (launch, combine
    # kernel; fitted to launches of 65 to 200 requests); negative: never.  Taken when the estimates
    # say so, which is when few sequences are left over (contexts of 4,096, 65 / 72 / 130 / 200 requests
    # of 4 kv heads: 96 / 107 / 188 / 283 us against 108 / 115 / 199 / 298 in one launch; 80 and 144: as
    # fast either way, one launch).
    many_second_launch_us: float = 9.0
    # single tokens of more pairs than CUs in a step that says how long its contexts are: shares of one
    # length for all sequences (a long sequence among short ones is cut into up to share_slots_growth times
    # the shares of the plan for equal contexts, no more than share_slots_waves wavefronts launched in all;
    # those a sequence does not use leave at once).  Off by default: it pays where contexts differ (7B
    # shape, 128 requests, us a layer: lengths uniform in 64..4,096 117 against 135, one request in eight at
    # 4,096 among short ones 77-87 against 131; 256 requests 112-161 against 184-240; a serving load of 128
    # in flight with prompts of 64 to 3,500 tokens: 5,288 against 5,230 tok/s, its steps being mostly
    # prompt portions) and costs where they are equal (a decode step of 96 / 128 / 256 requests at
    # contexts of 4,096: +2.9 / +1.0 / +7.5 %: more share slots to combine, and a combine kernel where one
    # share a pair needed none), which is what the decode benchmarks measure.
    shares_of_one_length: bool = False
    share_slots_growth: int = 4
    share_slots_waves: int = 4096
    # prompt launches share keys through LDS from this many 32-column wavefronts and this context
    # on (7B shape, laid out by chiplet, a workgroup per tile: as fast or faster than a wavefront
    # per 32 columns straight from the pages at every size measured, from 8 tokens to 32 k)
    shared_attention_min_waves: int = 0
    shared_attention_min_context: int = 0
    # a launch of unpaired tiles that does not start at the beginning of its contexts (a portion
    # deep in a prompt) has every tile cut into shares of its keys, a workgroup each: as many as
    # bring the launch to split_workgroups workgroups (7B shape: 512 tokens after 7,680, 112 tiles:
    # 223 / 135 / 108 / 116 us in 1 / 2 / 4 / 8 shares; 32 tokens after 4,064, 8 tiles: 118 us in one,
    # 23.5 in 16), from deep_blocks key blocks on at least split_deep (2,048 tokens after 30,720: 1,106
    # / 1,023 / 1,065 us in 1 / 4 / 8), at most split_max, none of fewer than min_blocks key blocks
    # (16 tokens after 2,032, 16 requests: 34 us with shares of 8 blocks, 46 us of 4), and no more
    # than keep the partial outputs below split_bytes
    prompt_split_workgroups: int = 512
    prompt_split_min_blocks: int = 8
    prompt_split_max: int = 32
    prompt_split_deep_blocks: int = 384
    prompt_split_deep: int = 4
    prompt_split_bytes: int = 512 << 20
    # a launch of whole prompts with fewer workgroups of 128 columns than this takes workgroups of 64
    # columns: a wavefront then holds 16 columns and three fit a SIMD (7B shape, one prompt, a workgroup
    # per tile: 2,048 tokens 57.5 against 71.4 us, 2,560: 78 against 86, 3,072: 113 against 102; portions
    # deep in a context keep 128 columns: 2,048 tokens after 6,144: 290 against 332 us)
    narrow_attention_workgroups: int = 600
    # ... and prompts of at most narrow_attention_short_tokens tokens up to narrow_attention_short_workgroups:
    # several short prompts have as many workgroups as one long one, but no long tiles for which the
    # wider workgroups' fewer reads of the keys would pay (us, 64 against 128 columns: 7B shape, four
    # prompts of 1,024 tokens 62 against 76; 32B shape, two of 1,024: 43 against 51, four: 80 against 85;
    # 72B shape, four of 1,024: 118 against 120; two prompts of 2,048 tokens take the same time either way)
    narrow_attention_short_tokens: int = 1024
    narrow_attention_short_workgroups: int = 2000
    # where the launch is not laid out by chiplet (3, 5, 6, 7, 9.. kv heads), a workgroup of a whole
    # prompt takes a late tile of the causal triangle and its early mirror, unless the pairs would
    # fill the chip (two workgroups a CU) in several rounds, the last of them mostly empty: below
    # this share of the slots of all rounds, every tile gets a workgroup of its own.  Laid out by
    # chiplet, a workgroup per tile, long tiles first, is as fast or faster everywhere (7B shape:
    # 1,536 tokens 44 against 57 us, 2,048: 57.5 against 70, 4,096: 168 against 178, 8,192: 537 against 613)
    pair_prompt_tiles: bool = True
    unpaired_below_fill: float = 0.9

    def apply(self, table) -> None:
        """Sets every field on ``table`` under its upper-case name."""
        for f in fields(self):
            setattr(table, f.name.upper(), getattr(self, f.name))
