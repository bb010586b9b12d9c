"""Position encodings of a mixer (tables, rotation and cache write, the q/k/v product that carries
them) and attention over the paged cache (matrix-core kernels per head size, the general kernel
for everything they refuse)."""
import ctypes

import torch

from . import build
from .values import (KernelError, LinearWeight, PartialSums, RotationPlan, ScaledRows, TiledRows,
                     _RopeStore, _c_float, _p, _ptr)


class AttentionOps:
    # ----------------------------------------------------------------- rope
    def rope_tables(self, positions, inv_freq):
        T, half = positions.shape[0], inv_freq.shape[0]
        self._check(positions, torch.int32, (T,), "positions")
        self._check(inv_freq, torch.float32, (half,), "inv_freq")
        cos = self._new((T, half), torch.float32)
        sin = self._new((T, half), torch.float32)
        self._call("elementwise", "sl_rope_tables", _p(positions), _p(inv_freq), _p(cos), _p(sin),
                   T, half)
        return cos, sin

    def _check_pages(self, k_cache, v_cache, nkv, D, page_size):
        pages = k_cache.shape[0]
        self._check(k_cache, self.act_dtype, (pages, nkv, page_size, D), "K pages")
        self._check(v_cache, self.act_dtype, (pages, nkv, D, page_size), "V pages")
        return pages

    def rope_store(self, qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                   pairs8=False, split=None, rot_dim=None, q_scale=1.0):
        """Rotate q and k of ``qkv`` in place (``cos`` None: no rotation) and write
        k and v to their cache rows (``k_cache`` None: no write).  The first
        ``rot_dim`` channels of a head are rotated (default: all), pair j being
        (j, j + rot_dim / 2); ``pairs8``: they come in blocks of 8 channels and
        their 8 partners (the order ``qkv_rope_store`` uses) instead.
        ``split``: the product arrives as ``PartialSums``; ``qkv`` is then only
        written (its q columns).  ``q_scale`` multiplies the q heads after the
        rotation, before their rounding."""
        T = qkv.shape[0]
        rot = D if rot_dim is None else int(rot_dim)
        if rot % 2 or not 0 <= rot <= D or (pairs8 and rot % 16) or (cos is not None and rot == 0):
            raise KernelError(f"rope_store: cannot rotate {rot} of {D} channels"
                              + (" in blocks of 8 pairs" if pairs8 else ""))
        self._check(qkv, self.act_dtype, (T, (nh + 2 * nkv) * D), "qkv")
        parts = bias = None
        if split is not None:
            parts, bias = split.parts, split.bias
            self._check(parts, torch.float32, (parts.shape[0], T, (nh + 2 * nkv) * D), "partial sums")
            if bias is not None:
                self._check(bias, torch.float32, ((nh + 2 * nkv) * D,), "bias")
        if cos is not None:
            self._check(cos, torch.float32, (T, rot // 2), "cos")
            self._check(sin, torch.float32, (T, rot // 2), "sin")
        if k_cache is not None:
            self._check_pages(k_cache, v_cache, nkv, D, page_size)
            self._check(slots, torch.int32, (T,), "slots")
        self._call("elementwise", "sl_rope_store", _p(qkv), _p(cos), _p(sin), _p(slots),
                   _p(k_cache), _p(v_cache), T, nh, nkv, D, rot, page_size, int(pairs8),
                   _p(parts), parts.shape[0] if parts is not None else 0, _p(bias), _c_float(q_scale))

    def qkv_rope_store(self, x, weight, bias, nh, nkv, D, cos, sin, slots, k_cache, v_cache,
                       page_size, rot_dim=None, q_scale=1.0):
        """q/k/v product, rotation and cache write.  The rows of ``weight`` (and
        ``bias``) hold every q and k head in the blocked pair order (``pairs8``
        above).  Returns the [T, (nh + 2 nkv) D] buffer whose q columns the
        attention reads.  For at most 16 rows and a tiled weight all of it is
        one kernel; k and v columns of the buffer are then not written."""
        if not isinstance(weight, LinearWeight):
            weight = LinearWeight(weight)
        M, K = x.shape
        N = weight.shape[0]
        rot = D if rot_dim is None else int(rot_dim)
        if N != (nh + 2 * nkv) * D or D % 16 or rot % 16 or not 0 <= rot <= D:
            raise KernelError("qkv_rope_store: weight rows must be (nh + 2 nkv) * D with D % 16 == 0, "
                              "the rotated width a multiple of 16")
        fused = (self.act_dtype == torch.bfloat16 and self.fuse_rope and 0 < M <= self._fused_rows(K)
                 and weight.tiled is not None and weight.shape == (N, K))
        if not fused:
            plan = None if isinstance(x, ScaledRows) else self._block_plan(M, N, K, weight)
            if plan:
                # K split over workgroups of the block kernel; the rotation kernel adds the partial sums up
                self._check(x, self.act_dtype, (M, K), "x")
                product = self.linear_block(x, weight, bias, ks=plan[0], partial=True, square=plan[1])
                qkv = self._new((M, N))
                self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                                True, split=product, rot_dim=rot, q_scale=q_scale)
                return qkv
            if (self._wide_from(K) <= M <= self._few_rows_limit(weight) and K % 32 == 0
                    and not isinstance(x, ScaledRows)):
                # K split over workgroups; the rotation kernel adds the partial sums up
                product = self.linear_mid(x, weight, bias, partial=True)
                if isinstance(product, PartialSums):
                    qkv = self._new((M, N))
                    self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                                    True, split=product, rot_dim=rot, q_scale=q_scale)
                    return qkv
                qkv = product
            elif (self.act_dtype == torch.bfloat16 and not isinstance(x, ScaledRows)
                    and M > self._few_rows_limit(weight)):
                # many rows: the library keeps the float32 sums, and the rotation kernel adds the
                # float32 bias, rotates and rounds once, exactly as the fused few-rows kernel does
                self._check(x, self.act_dtype, (M, K), "x")
                sums = self.library_sums(x, self.rows_of(weight), torch.float32)
                qkv = self._new((M, N))
                self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                                True, split=PartialSums(sums.unsqueeze(0), bias), rot_dim=rot,
                                q_scale=q_scale)
                return qkv
            else:
                qkv = self.linear(x, weight, bias)
            self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size, True,
                            rot_dim=rot, q_scale=q_scale)
            return qkv
        scaled = x if isinstance(x, ScaledRows) else None
        if scaled is None:
            self._check(x, self.act_dtype, None, "x")
        if bias is not None:
            self._check(bias, torch.float32, (N,), "bias")
        if cos is not None:
            self._check(cos, torch.float32, (M, rot // 2), "cos")
            self._check(sin, torch.float32, (M, rot // 2), "sin")
        if k_cache is not None:
            self._check_pages(k_cache, v_cache, nkv, D, page_size)
            self._check(slots, torch.int32, (M,), "slots")
        rope = _RopeStore(_ptr(cos), _ptr(sin), _ptr(slots if k_cache is not None else None),
                          _ptr(k_cache), _ptr(v_cache), nh, nkv, D, page_size, rot, q_scale)
        qkv = self._new((M, N))
        self._skinny(scaled.x if scaled is not None else x, weight, bias, qkv, M, N, K,
                     scaled=scaled, rope=rope)
        return qkv

    # --------------------------------------------- position encodings of a mixer
    def plan_rotation(self, head_dim, layout) -> RotationPlan:
        """The channel order of q and k heads for a position encoding whose
        ``layout`` is None (nothing is rotated) or says ``rot_dim`` (the leading
        channels that are rotated) and ``pairing``: "half" pairs channel j with
        j + rot_dim / 2, "interleaved" 2j with 2j + 1.  Scores do not depend on
        the order of the channels as long as q and the cached k agree, so an
        interleaved pairing is turned into halves by the order alone, and the
        rotated channels are laid out in blocks of 8 and their 8 partners where
        the fused q/k/v kernel can take them (head size and rotated width
        multiples of 16)."""
        D = int(head_dim)
        rot = 0 if layout is None else int(layout.rot_dim)
        pairing = "half" if layout is None else layout.pairing
        if rot % 2 or not 0 <= rot <= D:
            raise KernelError(f"a rotation of {rot} of {D} channels has no kernel: the width must be even")
        if pairing not in ("half", "interleaved"):
            raise KernelError(f"pairing '{pairing}' has no kernel (half or interleaved)")
        order = list(range(D))
        if pairing == "interleaved":
            order[:rot] = list(range(0, rot, 2)) + list(range(1, rot, 2))
        blocked = D % 16 == 0 and rot % 16 == 0
        if blocked and rot:
            halves = order[:rot]
            order[:rot] = [halves[(i % 16 >= 8) * (rot // 2) + 8 * (i // 16) + i % 8] for i in range(rot)]
        plain = order == list(range(D))
        return RotationPlan(None if plain else torch.tensor(order, dtype=torch.long), rot, blocked)

    LOG2E = 1.4426950408889634

    def split_attention_scale(self, scale: float):
        """(factor for q at its producer, scale left for ``paged_attention``).
        The matrix-core attention kernels want their scores in units of log 2:
        q then leaves ``project_qkv`` multiplied by scale * log2(e) (before its
        one rounding) and the attention call gets ln 2, whose product with
        log2(e) is 1, so no multiply-add per score is left.  The float32 table
        keeps the scale where the reference has it."""
        if self.act_dtype != torch.bfloat16 or not self.use_mfma_attention:
            return 1.0, float(scale)
        return float(scale) * self.LOG2E, 1.0 / self.LOG2E

    def project_qkv(self, x, weight, bias, nh, nkv, D, plan, tables, slots, k_cache, v_cache,
                    page_size, q_scale=1.0):
        """What a mixer calls: the q/k/v product of ``x`` (rows of ``weight`` in
        the order of ``plan``), the position encoding's work on q and k for this
        step's ``tables`` (whatever the encoding's ``tables()`` returned: None,
        or an object with ``cos`` and ``sin`` [T, rot_dim / 2]) and the write of
        k and v into the cache.  Returns [T, (nh + 2 nkv) D] whose q columns the
        attention reads, multiplied by ``q_scale`` (see ``split_attention_scale``)."""
        cos = sin = None
        if tables is not None:
            cos, sin = getattr(tables, "cos", None), getattr(tables, "sin", None)
            if cos is None or sin is None:
                raise KernelError(f"position tables of type {type(tables).__name__} have no kernel: "
                                  "this table rotates channel pairs by cos and sin and nothing else")
            if plan.rot_dim == 0:
                raise KernelError("the position encoding gives tables but its layout rotates nothing")
        if plan.blocked:
            return self.qkv_rope_store(x, weight, bias, nh, nkv, D, cos, sin, slots, k_cache, v_cache,
                                       page_size, rot_dim=plan.rot_dim, q_scale=q_scale)
        qkv = self.linear(x, weight, bias)
        self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                        rot_dim=plan.rot_dim, q_scale=q_scale)
        return qkv

    # ------------------------------------------------------------ attention
    def attend_and_project(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                           batch, scale, window, w_out, bias=None, defer=False):
        """``paged_attention`` followed by ``linear`` with the output projection.  For a step of a few
        single tokens the kernel table keeps what lies between them laid out by k-step, as
        ``gated_mlp`` does (at 16 rows the projection reads as many bytes of x as of W)."""
        if not isinstance(w_out, LinearWeight):
            w_out = LinearWeight(w_out)
        T = qkv.shape[0]
        tiled = (self.tile_few_rows and 1 < T <= self._fused_rows(w_out.shape[0]) and batch.max_q_len == 1
                 and batch.num_prefill_seqs == 0 and batch.num_seqs == T and w_out.tiled is not None
                 and w_out.shape[1] == nh * D
                 and self._mfma_attention_fits(D, nh // nkv, block_tables.shape[1], page_size, batch))
        attn = self.paged_attention(qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                                    batch, scale, window, _tiled_out=tiled)
        return self.linear(attn, w_out, bias, defer=defer)

    def paged_attention(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                        batch, scale, window, _tiled_out=False):
        T = qkv.shape[0]
        S, max_pages = block_tables.shape
        self._check(qkv, self.act_dtype, (T, (nh + 2 * nkv) * D), "qkv")
        self._check_pages(k_cache, v_cache, nkv, D, page_size)
        self._check(block_tables, torch.int32, None, "block tables")
        self._check(batch.tok_seq, torch.int32, (T,), "tok_seq")
        self._check(batch.positions, torch.int32, (T,), "positions")
        if S != batch.num_seqs:
            raise KernelError(f"block tables hold {S} sequences, the batch {batch.num_seqs}")
        if batch.max_ctx_len > max_pages * page_size:
            raise KernelError("block table is shorter than the context")
        out = self._new((T, nh * D))
        if self._mfma_attention_fits(D, nh // nkv, max_pages, page_size, batch):
            self._attention_mfma(qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                                 batch, scale, window, out, out_rows=T if _tiled_out else 0)
            return TiledRows(out, (T, nh * D)) if _tiled_out else out
        stride = (nh + 2 * nkv) * D
        first = 0                         # tokens before this one are done
        n_pre, n_pre_tok = batch.num_prefill_seqs, batch.num_prefill_tokens
        if n_pre and D % 16 == 0 and batch.max_q_len > 1:
            # prompt portions (they come first in the batch): workgroups that stage each block of keys
            # once for 16 columns, instead of a wavefront per (token, head) that reads its own
            self._check(batch.cu_q, torch.int32, (batch.num_seqs + 1,), "cu_q")
            self._call("attention", "sl_attention_general_tiles", _p(qkv), stride, _p(k_cache),
                       _p(v_cache), _p(block_tables), max_pages, _p(batch.cu_q), _p(batch.positions),
                       n_pre, batch.max_q_len, nh, nkv, D, page_size, _c_float(scale),
                       int(window or 0), _p(out))
            first = n_pre_tok
        rest = T - first
        if rest == 0:
            return out
        # few tokens (a decode step): the keys of every (token, head) are shared out over several
        # wavefronts; the count depends on the number of tokens only, so that a captured step and an
        # eager one add up in the same order
        single = first > 0 or batch.max_q_len == 1
        group = nh // nkv                 # a wavefront takes up to 8 heads of a group together
        per_token = nkv * -(-group // 8) if group > 1 else nh
        nsplit = max(1, min(64, self.GENERAL_ATTENTION_WAVES // (rest * per_token))) if single else 1
        part_o = part_ml = None
        if nsplit > 1:
            part_o = self._new((rest, nh, nsplit, D), torch.float32)
            part_ml = self._new((rest, nh, nsplit, 2), torch.float32)
        self._call("attention", "sl_attention_general", _p(qkv[first:]), stride, _p(k_cache),
                   _p(v_cache), _p(block_tables), max_pages, _p(batch.tok_seq[first:]),
                   _p(batch.positions[first:]), rest, nh, nkv, D, page_size, _c_float(scale),
                   int(window or 0), _p(out[first:]), nsplit, _p(part_o), _p(part_ml))
        return out

    def _mfma_attention_fits(self, D, group, max_pages, page_size, batch):
        """The matrix-core kernels take bfloat16, head sizes that are multiples
        of 32, and block tables that cover the context rounded up to a whole
        32-key block; everything else goes to the general kernel."""
        if self.act_dtype != torch.bfloat16 or not self.use_mfma_attention:
            return False
        if D % 32 or D > 256 or group > 64:
            return False
        return max_pages * page_size >= -(-batch.max_ctx_len // 32) * 32

    def _attention_lib(self, D):
        key = ("attention_mfma", D)
        lib = self._lib.get(key)
        if lib is None:
            lib = build.load(build.unit("attention_mfma", "bfloat16", SL_HEAD_DIM=D))
            self._lib[key] = lib
        return key

    def _decode_shares(self, units, most, blocks, D) -> int:
        """Into how many shares the ``blocks`` key blocks of each of ``units`` (request, kv head) pairs, no
        more pairs than CUs, are cut, ``most`` at most: the count with the lowest estimate of the launch's
        time, fewest shares first among equals.  A share is a wavefront; it asks for two blocks at a time,
        so its keys take ceil(blocks of the longest share / 2) trips to memory (FEW_TRIP_US each), unless
        the stream of all keys and values through the fullest CU takes longer (a launch takes what its
        busiest CU holds: 7B shape, contexts of 4,096, 14 requests in 10 shares, 560 wavefronts on 256
        CUs: 30.6 us a layer; in 9, 504 wavefronts: about 22 us); every wavefront a CU costs FEW_WAVE_US,
        and the combine kernel reads the partial results sixteen shares at a time, FEW_BATCH_US a batch.
        Fitted to 1,500 launches of 1 to 24 requests of the 7B shape at contexts of 512 to 32,768 (mean
        error 4 %); over those and four further contexts the count taken costs 0.5 % more than the best
        measured one on average and 4 % at worst.
        (Filling whole rounds of the CUs near two wavefronts each, the rule before: 1.2 % and 20 %: it took
        128 shares for one request at 8,192 to 16,384 keys where 64 are faster, 12.0 against 10.2 us, and
        fewer than the context allows at 512 and 1,024 keys, where one trip beats full rounds.)"""
        cus = self._num_cus
        stream = units * blocks * 32 * D * 4 / (self.FEW_STREAM_GBS_PER_CU * 1e3 * cus)       # us for K and V
        best, lowest = 1, None
        for shares in range(1, max(1, min(most, 8 * cus // units)) + 1):
            waves = units * shares
            trips = -(-(-(-blocks // shares)) // 2)
            t = max(self.FEW_TRIP_US * trips, stream * (-(-waves // cus) * cus / waves)) + self.FEW_WAVE_US * waves / cus
            if shares > 1:
                t += self.FEW_BATCH_US * -(-shares // 16) + self.MANY_COMBINE_US
            if lowest is None or t < lowest - 1e-9:
                best, lowest = shares, t
        return best

    def _decode_many(self, pairs, blocks, D, merged_fits, most):
        """(merged in the workgroup, shares) for single-token rows of more (request, kv head) pairs than
        CUs, by the estimate of the launch's time that ``Tuning.many_*`` describes.  Wavefronts of a share
        each all have to be on the chip at once (eight a CU), or the launch runs in two waves of them."""
        cus = self._num_cus
        stream = pairs * blocks * 32 * D * 4 / (self.MANY_STREAM_GBS_PER_CU * 1e3 * cus)      # us for K and V

        def rounds(units):                           # as if every CU had as many units as the fullest
            return -(-units // cus) * cus / units

        def fullest(waves):
            return rounds(waves) if waves <= self.MANY_CROWDED_WAVES * cus else 1 + self.MANY_CROWDED * (rounds(waves) - 1)

        forms = []                                   # (estimate, merged, shares), fewest shares first
        if merged_fits:
            forms.append((stream * (1 + self.MANY_MERGED_ROUNDS * (rounds(pairs) - 1)) * self.MANY_MERGED_BASE, True, 1))
        for k in range(1, max(1, min(most, 8 * cus // pairs)) + 1):
            t = max(-(-blocks // (2 * k)) * self.MANY_TRIP_US, stream * fullest(pairs * k)) + self.MANY_SHARE_US * k
            forms.append((t + (self.MANY_COMBINE_US if k > 1 else 0.0), False, k))
        lowest = min(t for t, _, _ in forms)
        estimate, merged, shares = next(f for f in forms if f[0] <= self.MANY_FEWER_WITHIN * lowest)
        return merged, shares, estimate

    def _decode_launches(self, n_dec, nkv, blocks, D, merged_fits, most):
        """The launches over the single-token rows of a step: (first sequence, sequences, merged in
        the workgroup, shares) each.  With a (request, kv head) pair for every CU, a workgroup of
        eight wavefronts takes a pair: its wavefronts cut the keys among themselves and merge in LDS,
        no partial results in memory and no second kernel.  With fewer pairs that would leave a
        pair's keys to the one CU that runs its workgroup, and a CU pulls 50 GB/s whatever is in
        flight (7B shape, contexts of 4,096, 8 requests: 61 us against 16 us): then a wavefront of a
        workgroup of its own takes a share, as many shares as ``_decode_shares`` estimates to be
        fastest, spread over all CUs, and the combine kernel merges them (a few requests with long
        contexts: up to 256 shares; one request at 32,000 tokens: 128).  The shorter the contexts, the
        fewer pairs it takes for merging in the workgroup to pay (``Tuning.group_attention_from``).
        More pairs than CUs: one launch in the form ``_decode_many`` estimates to be the fastest, or two, the sequences that fill whole rounds of
        the CUs merged in the workgroup and the others as a launch of few pairs, if the estimates say
        that is faster (the first launch then runs at the rate of a stream, whatever the number of
        sequences)."""
        pairs, cus = n_dec * nkv, self._num_cus

        def few(n):
            share = next(s for b, s in self.GROUP_ATTENTION_FROM if blocks <= b)
            merged = merged_fits and n * nkv >= self.GROUP_ATTENTION_FILL * share * cus
            return merged, 1 if merged else self._decode_shares(n * nkv, min(most, blocks // 2), blocks, D)

        if pairs <= cus:
            return [(0, n_dec) + few(n_dec)]
        merged, shares, estimate = self._decode_many(pairs, blocks, D, merged_fits, min(most, blocks // 2))
        per_round = cus // nkv
        rest = n_dec % per_round if cus % nkv == 0 else 0
        if merged_fits and rest and self.MANY_SECOND_LAUNCH_US >= 0:
            stream = lambda n: n * nkv * blocks * 32 * D * 4 / (self.MANY_STREAM_GBS_PER_CU * 1e3 * cus)
            m2, k2 = few(rest)
            each = 8 if m2 else k2                    # wavefronts a pair
            waves = rest * nkv * each
            second = max(-(-blocks // (2 * each)) * self.MANY_TRIP_US, stream(rest) * (-(-waves // cus) * cus / waves))
            if stream(n_dec - rest) + second + self.MANY_SECOND_LAUNCH_US < estimate:
                return [(0, n_dec - rest, True, 1), (n_dec - rest, rest, m2, k2)]
        return [(0, n_dec, merged, shares)]

    def _pair_prompt_tiles(self, tiles, prompts_and_heads) -> bool:
        """Whether the workgroups of a whole prompt's attention take a late tile of the causal triangle and
        its early mirror (equal work for all, half as many workgroups) or a tile each, long ones first;
        asked only for launches that are not laid out by chiplet, which always take a tile each.
        Equal workgroups fill the chip in rounds of two per CU, and the last round may be nearly empty;
        tiles of their own leave the balance to the order in which workgroups start, at the price of
        twice the prologues.  7B shape, one prompt, pairs against a tile each: 4,096 tokens (448 pairs, one
        round) 175 against 223 us, 5,120 (560) 335 against 270, 7,168 (784) 546 against 461, 8,192 (896) 615
        against 572, 10,240 (1,120) 972 against 880, 14,336 (1,568) 1,842 against 1,618, 16,384 (1,792: three
        and a half rounds) 2,040 either way."""
        if not self.PAIR_PROMPT_TILES:
            return False
        pairs = -(-tiles // 2) * prompts_and_heads
        slots = 2 * self._num_cus
        rounds = -(-pairs // slots)
        return rounds == 1 or pairs >= self.UNPAIRED_BELOW_FILL * rounds * slots

    def _attention_mfma(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables, batch,
                        scale, window, out, out_rows=0):
        lib = self._attention_lib(D)
        self._check(batch.cu_q, torch.int32, (batch.num_seqs + 1,), "cu_q")
        max_pages = block_tables.shape[1]
        n_pre, n_pre_tok = batch.num_prefill_seqs, batch.num_prefill_tokens
        n_dec = batch.num_seqs - n_pre
        if n_dec and n_pre_tok + n_dec != batch.num_tokens:
            raise KernelError("single-token sequences must come last in the batch")
        common = (_p(qkv), (nh + 2 * nkv) * D, _p(k_cache), _p(v_cache), _p(block_tables),
                  max_pages, _p(batch.cu_q), _p(batch.positions))
        tail = (nh, nkv, D, page_size, _c_float(scale), int(window or 0))
        name = f"sl_attention_mfma@{D}"
        if name not in self._fn:
            fn = self._lib[lib].sl_attention_mfma
            fn.restype = ctypes.c_char_p
            self._fn[name] = fn
        if n_pre:
            waves = -(-batch.max_q_len * (nh // nkv) // 32) * nkv * n_pre
            shared = (waves >= self.SHARED_ATTENTION_MIN_WAVES and
                      batch.max_ctx_len >= self.SHARED_ATTENTION_MIN_CONTEXT and
                      bool(self._lib[lib].sl_attention_mfma_shares_keys()))
            tiles = -(-batch.max_q_len * (nh // nkv) // 128) * nkv * n_pre      # workgroups of 128 columns
            # tiles of a causal triangle differ in length; those of a portion that starts deeper in
            # its context than it is long do not
            triangle = batch.max_ctx_len < 2 * batch.max_q_len
            by_chiplet = bool(self._lib[lib].sl_attention_mfma_by_chiplet(nkv))
            pair = (triangle and not by_chiplet and
                    self._pair_prompt_tiles(-(-batch.max_q_len * (nh // nkv) // 128), nkv * n_pre))
            # few tiles over a long context: each is cut into shares of its keys
            nsplit, part_o, part_ml = 1, None, None
            if shared and not triangle:
                blocks = batch.max_ctx_len // 32
                nsplit = self.PROMPT_SPLIT_WORKGROUPS // tiles
                if blocks >= self.PROMPT_SPLIT_DEEP_BLOCKS:
                    nsplit = max(nsplit, self.PROMPT_SPLIT_DEEP)
                nsplit = max(1, min(nsplit, self.PROMPT_SPLIT_MAX, blocks // self.PROMPT_SPLIT_MIN_BLOCKS,
                                    int(self._lib[lib].sl_attention_mfma_max_splits()),
                                    self.PROMPT_SPLIT_BYTES // (n_pre_tok * nh * D * 4)))
            if nsplit > 1:
                part_o = self._new((n_pre_tok, nh, nsplit, D), torch.float32)
                part_ml = self._new((n_pre_tok, nh, nsplit, 2), torch.float32)
            # workgroups of 64 columns instead of 128 for launches below this many of the latter
            narrow_below = (self.NARROW_ATTENTION_SHORT_WORKGROUPS if batch.max_q_len <= self.NARROW_ATTENTION_SHORT_TOKENS
                            else self.NARROW_ATTENTION_WORKGROUPS)
            self._call(lib, name, *common, 0, n_pre, batch.max_q_len, *tail, nsplit,
                       0 if shared else 1 << 30, int(pair), _p(out), _p(part_o), _p(part_ml), 0,
                       n_pre_tok if nsplit > 1 else 0, narrow_below if triangle else 0, 0, 0, None, 0)
        if n_dec:
            blocks = -(-batch.max_ctx_len // 32)
            if window:
                blocks = min(blocks, -(-int(window) // 32) + 1)
            most = int(self._lib[lib].sl_attention_mfma_max_splits())
            fits = nh // nkv <= int(self._lib[lib].sl_attention_mfma_group_heads())
            launches = self._decode_launches(n_dec, nkv, blocks, D, fits, most)
            # (Tuning.shares_of_one_length) More pairs than CUs in one launch, and the step says how long its
            # contexts are: shares of one length for all its sequences (see share_count in the kernel).  The launch is planned as for
            # equal contexts, in shares (workgroups that merge in LDS wait for their longest sequence), aims
            # at the wavefronts of that plan, and has room for SHARE_SLOTS_GROWTH times as many shares of a
            # long sequence among short ones (up to SHARE_SLOTS_WAVES wavefronts launched in all).  7B shape,
            # 128 requests, us a layer: contexts of 4,096 all 174 (173 in two shares each); uniform in 64..4,096:
            # 117 against 135; one in eight at 4,096 and the others below 512: 77-87 against 131.  With fewer
            # pairs the plans above are as good or better (64 requests, uniform: 79 against 71 merged).
            stats = getattr(batch, "ctx_stats", None) if self.SHARES_OF_ONE_LENGTH else None
            if stats is not None and len(launches) == 1 and n_dec * nkv > self._num_cus:
                shares = launches[0][3] if not launches[0][2] else \
                    self._decode_many(n_dec * nkv, blocks, D, False, min(most, blocks // 2))[1]
                room = min(self.SHARE_SLOTS_GROWTH * shares, self.SHARE_SLOTS_WAVES // (n_dec * nkv))
                slots = max(1, min(most, max(1, blocks // 2), max(shares, room)))
                launches = [(0, n_dec, False, slots)] if slots > 1 else launches
                aim = shares * n_dec * nkv if slots > 1 else 0
            else:
                aim = 0
            for first, count, group, nsplit in launches:
                part_o = part_ml = None
                if nsplit > 1:
                    part_o = self._new((count, nh, nsplit, D), torch.float32)
                    part_ml = self._new((count, nh, nsplit, 2), torch.float32)
                self._call(lib, name, *common, n_pre + first, count, 1, *tail, nsplit, 0, 0, _p(out),
                           _p(part_o), _p(part_ml), n_pre_tok + first, count if nsplit > 1 else 0, 0,
                           int(out_rows), int(group), _p(stats) if aim else None, aim)
