"""Prefill operator: owns the compiled kernel variants of one AttentionEngine and launches them.

Host-side counterpart of the reference's generated ``_attention.forward`` + ``tl.compile`` result
(attention_engine/core/template/tl_template/attn/attn_tl.py:523-528, 567-580; block-sparse:
blockattn_tl.py:401-447): takes q/k/v ``[B,S,H,D]`` plus the CustomIO tensors (and, when a block
mask is in play, that mask as the LAST positional argument), allocates ``o`` and the final
rowscales, launches on torch's current stream, returns ``o``.
"""
from __future__ import annotations

import os

import torch

from ..runtime import hip_rt as rt
from ..transform.core import _convert_mask_to_block_mask, is_causal_mask
from . import lower as L
from .mask import plan_mask


def _dim(x, default):
    return default if isinstance(x, str) else int(x)


class PrefillOp:
    MASK_ROWS_PER_TILE = 8      # block-mask rows one q tile may span (AE_TT_ROWS of csrc/kernels/ae_tile_table.h)

    def __init__(self, qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func, mask_value,
                 infer_mask=True, infer_mask_block_M=128, infer_mask_block_N=128,
                 extern_block_mask=False, split_kv=False, target_workgroups=256,
                 tiles=None, tune=False, tune_file="", tune_bwd=False, tune_file_bwd="",
                 exact_scale=None, defer_norm=None, allow_spills=None):
        self._ctor = ((qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func, mask_value),
                      dict(infer_mask=infer_mask, infer_mask_block_M=infer_mask_block_M,
                           infer_mask_block_N=infer_mask_block_N, extern_block_mask=extern_block_mask,
                           split_kv=split_kv, target_workgroups=target_workgroups,
                           exact_scale=exact_scale, defer_norm=defer_norm, allow_spills=allow_spills))
        # numerics switches (see AttentionEngine): None = the default of the kernel / lowering
        self.exact_scale = exact_scale
        # None: a build that moves register tuples through scratch memory is reported, False: it is refused
        # (hip_rt.check_spills); where the pipelined kernel was this operator's own choice it then gives way to the
        # generic one, see _gives_way_to_the_generic_kernel
        self.allow_spills = allow_spills
        self._tiles_given = tiles is not None
        q_meta, k_meta, v_meta = qkv_meta
        self.dtype = q_meta.dtype
        self.D = int(q_meta.shape[3])
        self.DV = int(v_meta.shape[3])
        if int(k_meta.shape[3]) != self.D:
            raise ValueError("q and k head dims differ")
        if self.D % 16 or self.DV % 32:
            raise NotImplementedError(f"head dims (D={self.D}, DV={self.DV}) must be multiples of 16 / 32")
        # Value head dim 512 with head dim 64 / 128 / 256 (attn_script/retention.py: D 256, DV 512) runs in one
        # launch of the direct-to-LDS kernel: 256 accumulator registers per lane, one wave per SIMD, its
        # epilogue working block by block.  Other value head dims above 256 run as several launches over
        # column slices of V and of the output (the scores are recomputed per slice; the row scales of every
        # launch are the same); AE_DV_SLICE=1 forces that form.
        self.DV_launch = self.DV
        single_pass = (self.D in (64, 128, 256) and self.DV == 512 and os.environ.get("AE_DV_SLICE", "") != "1"
                       and not split_kv)
        if self.DV > 256 and not single_pass:
            self.DV_launch = next(c for c in (256, 192, 128, 96, 64, 32) if self.DV % c == 0)
        self.mask_mod = mask_mod
        self.elementwise_mask = mask_mod is not None and mask_value == "-inf"
        self.mask_value_zero = mask_value == "0"
        self.extern_block_mask = bool(extern_block_mask)
        self.mask_block = (int(infer_mask_block_M), int(infer_mask_block_N))
        self.functors = L.trace_functors(score_mod, mask_mod, online_func, custom_fwd_inputs,
                                         self.dtype, mask_value, defer_norm=defer_norm)
        self._graph = (score_mod, online_func, custom_fwd_inputs)     # the backward traces score_mod again
        self.functor_src = L.render_functors(self.functors)
        # what the software-pipelined kernel can run: the proven online softmax, or an elementwise graph
        # (masked scores are -inf before score_mod there, as in the reference: not with mask_value "0")
        self._pipe_softmax = None if self.mask_value_zero else self.functors.softmax
        self._pipe_elementwise = (self._pipe_softmax is None and self.functors.elementwise
                                  and not self.mask_value_zero)
        self.tiles = L.choose_prefill_tiles(self.D, self.DV_launch, _dim(q_meta.shape[2], 0),
                                            self._pipe_softmax,
                                            _dim(q_meta.shape[0], 1) * _dim(q_meta.shape[1], 1),
                                            elementwise=self._pipe_elementwise,
                                            seqlen_kv=_dim(k_meta.shape[2], 0))
        # Masks that reach the kernel as a tile table (anything but none / exactly causal) go to the generic
        # kernel: with its 128-row q tiles fewer tiles are partly visible, and its masked path costs less than
        # the pipelined kernel's (B2 H32 S4096 D128, sliding window of 256: 0.13 against 0.31 ms; a random block
        # mask that keeps 27 %: 0.22 against 0.35 ms).  tune=True still measures both.
        if self.tiles.rows_per_wave == 64 and os.environ.get("AE_PREFILL_KERNEL", "") != "pipelined" and (
                self.extern_block_mask or (mask_mod is not None and self._probe_mask_mode(q_meta, v_meta) == 2)):
            self.tiles = L.PrefillTiles()
        # tune=True (attn_tl.py:465-521 of the reference): the tile configuration comes from the record of
        # this problem in tune_file, or is measured at the first call and recorded there.  Launches whose
        # tiles are bound to something else (split-KV, an external block mask) keep the fixed choice.
        self._tune_file, self._tune_pending, self.tune_times = "", False, None
        self._tune_bwd = (bool(tune_bwd), tune_file_bwd)
        if tiles is not None:
            self.tiles = tiles
        elif tune and tune_file and not split_kv and not extern_block_mask:
            from . import tuner
            self._tune_file = tune_file
            self._tune_keys = tuner.problem_keys(q_meta.shape, self.D, self.DV)
            found = tuner.decode_tiles(tuner.lookup(tune_file, self._tune_keys), self._tune_candidates())
            if found is not None:
                self.tiles = found
            else:
                self._tune_pending = True
        # Split-KV ("MHA decode": a few query tokens against a long KV, attn_engine.py:273-290 and
        # core/lower/lower_decode.py:287-313 of the reference): the kv axis is shared out over several
        # workgroups per q tile and the partial results are merged with the user's combine().
        self.split_kv = bool(split_kv)
        self.target_workgroups = int(target_workgroups)
        if self.split_kv:
            if self.tiles.template == "ae_prefill_simple.hip" or max(self.D, self.DV) > 128:
                raise NotImplementedError("split-KV prefill needs head dims 64 or 128")
            if self.DV_launch != self.DV:
                raise NotImplementedError("split-KV prefill with a value head dim above 256")
            if not hasattr(online_func, "combine"):
                raise NotImplementedError("split-KV needs OnlineFunc.combine to merge the partial results")
            from .lower_decode import lower_combine
            self.tiles = L.PrefillTiles()          # the generic kernel carries the split-KV mode
            self.functor_src += lower_combine(online_func, self.functors.final_rowscale_names)
        if self.extern_block_mask and self.tiles.rows_per_wave != 32 and (
                self.mask_block[1] % self.tiles.block_n or
                (self.tiles.block_m % self.mask_block[0] and self.mask_block[0] % self.tiles.block_m)):
            self.tiles = L.PrefillTiles()     # the pipelined kernel's kv tile is fixed; use the generic one
        if self.extern_block_mask:
            # a q tile covers whole block-mask rows, a kv tile sits inside one block-mask column
            while self.tiles.block_n > self.mask_block[1] and self.tiles.block_n > 32:
                self.tiles.block_n //= 2
            if self.tiles.block_m > self.MASK_ROWS_PER_TILE * self.mask_block[0]:
                self.tiles = L.PrefillTiles(block_n=self.tiles.block_n)   # 128-row q tiles span fewer table rows
            if (self.tiles.block_m % self.mask_block[0] and self.mask_block[0] % self.tiles.block_m) or \
                    self.mask_block[1] % self.tiles.block_n or \
                    self.tiles.block_m > self.MASK_ROWS_PER_TILE * self.mask_block[0]:
                raise NotImplementedError(f"block mask granularity {self.mask_block} does not fit the tiles")
        self.n_rowscales = len(self.functors.final_rowscale_names)
        if self.n_rowscales > rt.AE_MAX_ROWSCALES or len(self.functors.customs) > rt.AE_MAX_CUSTOM:
            raise NotImplementedError("too many rowscales / custom inputs")
        self.final_rowscales = {}
        self.block_mask = None
        self._variants = {}   # (mask_mode, even_q, even_kv) -> (module, cfg, config_src)
        self._plans = {}      # (B|1, H|1, Sq, Skv) -> MaskPlan with device table
        self.meta_shape = (_dim(q_meta.shape[0], 1), _dim(q_meta.shape[1], 1), _dim(q_meta.shape[2], 0),
                           _dim(v_meta.shape[2], 0))
        # compile for the declared shape now (hipRTC needs no GPU) so construction reports
        # lowering/compile errors, like the reference's constructor does
        B, H, Sq, Skv = self.meta_shape
        self.source = self.functor_src
        if Sq > 0:
            try:
                self._compile_declared_shape(B, H, Sq, Skv, infer_mask, mask_mod)
            except rt.SpillError:
                if not self._gives_way_to_the_generic_kernel():
                    raise
                self._compile_declared_shape(B, H, Sq, Skv, infer_mask, mask_mod)

    def _gives_way_to_the_generic_kernel(self) -> bool:
        """A build of the software-pipelined kernel that spills registers is refused (hip_rt.check_spills).  Where
        that kernel was this operator's own choice -- not the caller's (``tiles=``, the tuner) -- the operator
        switches to the generic kernel, whose two waves per SIMD leave the compiler room, for every later launch:
        True if it did.  (The pipelined kernel holds 64 query rows per wave in one wave per SIMD and fills the
        register file; its fp16 builds fit, some bf16 builds at head dim 128 spill a few values.)"""
        if self._tiles_given or self.tiles.template != "ae_prefill_pipe.hip":
            return False
        self.tiles = L.PrefillTiles()
        self._variants.clear()
        self._plans.clear()
        self._bwd = None            # (the backward reads this operator's mask plans: built again on demand)
        self.gave_way_to_generic = True
        return True

    def _compile_declared_shape(self, B, H, Sq, Skv, infer_mask, mask_mod):
        plan = self._plan(B, H, Sq, Skv, device=None)
        mode = 2 if self.extern_block_mask else plan.mode
        n_split, _ = self.plan_splits(B, H, Sq, Skv)
        _, _, cfg_src = self._variant(mode, Sq % self.tiles.block_m == 0, Skv % self.tiles.block_n == 0, n_split,
                                      self._table_rows(self.mask_block[0] if self.extern_block_mask else plan.block_m),
                                      plan.heavy_last and not self.extern_block_mask)
        self.source = cfg_src + "\n" + self.functor_src
        if infer_mask and mask_mod is not None and not self.extern_block_mask:
            self.block_mask = self._reference_block_mask(B, H, Sq, Skv)

    def _probe_mask_mode(self, q_meta, v_meta):
        """Mode of the mask plan at the declared sequence lengths (4096 where they are dynamic), for batch entry
        and head 0: 2 = the mask needs a tile table."""
        sq, skv = _dim(q_meta.shape[2], 4096), _dim(v_meta.shape[2], 4096)
        return plan_mask(self.mask_mod, self.functors.mask, 1, 1, sq, skv, 128, 64,
                         elementwise=self.elementwise_mask).mode

    # ---- tuning ------------------------------------------------------------------------
    def _tune_candidates(self):
        from . import tuner
        return tuner.prefill_candidates(self.D, self.DV_launch, self._pipe_softmax, self._pipe_elementwise)

    def _tune(self, q, k, v, *extra):
        """Measures every candidate tile configuration on the caller's tensors, becomes the fastest one and
        records it under this engine's problem keys (AE_TUNE_VERBOSE=1 prints the measurements)."""
        from . import tuner
        self._tune_pending = False
        args, kw = self._ctor
        log = print if os.environ.get("AE_TUNE_VERBOSE", "") == "1" else None
        cands = self._tune_candidates()
        mine = self.block_mask      # the engine appends this very object to every call: see _forward

        def run(o):
            return o._forward(q, k, v, *[o.block_mask if (mine is not None and x is mine) else x for x in extra])
        best, op, times = tuner.pick(
            cands, lambda t: self if t == self.tiles else PrefillOp(*args, **kw, tiles=t), run, log)
        if op is not self:
            keep = (self._ctor, self._tune_file, self._tune_keys, self._tune_bwd, mine)
            self.__dict__.update(op.__dict__)
            self._ctor, self._tune_file, self._tune_keys, self._tune_bwd, self.block_mask = keep
            self._bwd = None        # the backward reads this operator's mask plans: built again on demand
        self._tune_pending = False
        self.tune_times = {tuple(tuner.encode_tiles(cands[i])): ms for i, ms in times.items()}
        tuner.store(self._tune_file, self._tune_keys, tuner.encode_tiles(best))

    # ---- mask --------------------------------------------------------------------------
    def _plan(self, B, H, Sq, Skv, device):
        key = (B, H, Sq, Skv)
        plan = self._plans.get(key)
        if plan is None:
            plan = plan_mask(self.mask_mod, self.functors.mask, B, H, Sq, Skv, self.tiles.block_m,
                             self.tiles.block_n, elementwise=self.elementwise_mask)
            self._plans[key] = plan
        if device is not None and plan.table is not None and plan.table.device != device:
            plan.table = plan.table.to(device)
        return plan

    def _reference_block_mask(self, B, H, Sq, Skv):
        """The block mask the reference would keep on ``mod.block_mask`` (lower.py:721-738):
        int8 [B,H,Sq/bm,Skv/bn] "any element visible", or None when it is exactly block-causal
        (dense template)."""
        bm, bn = self.mask_block
        lm = self.functors.mask
        mb, mh = (B if lm.uses_b else 1), (H if lm.uses_h else 1)
        rows = []
        kv = torch.arange(Skv).view(1, 1, 1, Skv)
        for r0 in range(0, Sq, bm * 8):
            r1 = min(Sq, r0 + bm * 8)
            q = torch.arange(r0, r1).view(1, 1, -1, 1)
            m = self.mask_mod(torch.arange(mb).view(mb, 1, 1, 1), torch.arange(mh).view(1, mh, 1, 1), q, kv)
            if not isinstance(m, torch.Tensor):
                m = torch.tensor(bool(m))
            m = m.to(torch.bool).expand(mb, mh, r1 - r0, Skv)
            rows.append(_convert_mask_to_block_mask(m, bm, bn)[0])
        blocks = torch.cat(rows, dim=2).expand(B, H, -1, -1)
        if Sq == Skv and bool(is_causal_mask(blocks, bm, bn)):
            return None
        return blocks.contiguous()

    # ---- kernels -------------------------------------------------------------------------
    COMBINE_THREADS = 128

    def plan_splits(self, B, Hq, Sq, Skv):
        """(number of KV splits, kv positions per split): a workgroup for every CU of the chip (more splits cost
        more in partial results and their merge than they gain: B1 H32 Sq128 Skv8192, the shape of
        attn_script/mha_inference.py, 43 us with 8 splits, 44 with 16, 75 with 32), whole kv tiles per split, no
        empty split."""
        if not self.split_kv:
            return 1, Skv
        bn = self.tiles.block_n
        kv_tiles = -(-Skv // bn)
        wgs = -(-Sq // self.tiles.block_m) * (-(-(B * Hq) // 8) * 8)
        want = max(1, min(kv_tiles, -(-self.target_workgroups // wgs)))
        per = -(-kv_tiles // want)
        return -(-kv_tiles // per), per * bn

    def _kv_custom_scratch(self) -> int:
        """LDS a launch needs beyond its K / V stages: the direct-to-LDS kernel redistributes the tiles of custom
        inputs with a kv dimension (fetched in a coalesced layout) through 2560 bytes per wave and 32-row block
        (AE_KV_SCRATCH of ae_prefill.hip; its builds with two waves per SIMD)."""
        if (self.tiles.template != "ae_prefill.hip" or self.tiles.waves_per_eu < 2
                or not any(c.per_kv for c in self.functors.customs)):
            return 0
        return self.tiles.n_waves * (self.tiles.rows_per_wave // 32) * 2560

    def _clock_stamps(self):
        """AE_CLOCK_STAMPS=1 (a measurement switch, read by ``bench.py --mfma-probe``): the pipelined kernel is
        built so that every workgroup reports the shader-clock cycles and the 100 MHz ticks it ran for; the
        pairs of the last launch are kept on ``self.clock_stamps`` (int64 [workgroups, 2])."""
        return os.environ.get("AE_CLOCK_STAMPS", "") == "1" and self.tiles.template == "ae_prefill_pipe.hip"

    def _table_rows(self, mask_block_m):
        """Block-table rows a q tile spans (1, 2, 4 or 8): the kernels keep that many pairs of 64-bit masks."""
        if not mask_block_m:
            return 1
        rows = max(1, -(-self.tiles.block_m // int(mask_block_m)))
        return next(r for r in (1, 2, 4, 8) if r >= min(rows, 8))

    def _variant(self, mask_mode, even_q, even_kv, n_split=1, table_rows=1, heavy_last=False):
        if mask_mode != 2:
            table_rows, heavy_last = 1, False
        key = (mask_mode, even_q, even_kv, n_split, table_rows, bool(heavy_last))
        v = self._variants.get(key)
        if v is None:
            has_mask_mod = self.elementwise_mask and mask_mode != 1
            cfg_src = L.render_config(self.D, self.DV_launch, self.dtype, self.tiles, mask_mode, has_mask_mod,
                                      self.n_rowscales, self.functors.o_scale_one, even_q, even_kv,
                                      self._pipe_softmax if self.tiles.rows_per_wave == 64 else None,
                                      elementwise=self._pipe_elementwise and self.tiles.rows_per_wave == 64,
                                      exact_scale=self.exact_scale)
            if self.mask_value_zero:
                cfg_src += "#define AE_MASK_VALUE_ZERO 1\n"
            if mask_mode == 2:
                cfg_src += f"#define AE_TT_ROWS {table_rows}\n#define AE_HEAVY_LAST {1 if heavy_last else 0}\n"
            if n_split > 1:
                cfg_src += f"#define AE_NSPLIT {n_split}\n#define AE_COMBINE_THREADS {self.COMBINE_THREADS}\n"
            if self._clock_stamps():
                cfg_src += "#define AE_CLOCK_STAMPS 1\n"
            module = rt.compile_module(self.tiles.template, {"ae_config.h": cfg_src,
                                                          "ae_functors.h": self.functor_src},
                                       allow_spills=self.allow_spills,
                                       # the builds in which a spilled tuple came back wrong: 256 accumulator registers
                                       strict_spills=self.tiles.template == "ae_prefill.hip" and self.DV_launch > 256)
            cfg = rt.TileCfg(block_m=self.tiles.block_m, block_n=self.tiles.block_n,
                             threads=64 * self.tiles.n_waves,
                             lds_bytes=self.tiles.lds_bytes(self.D, self.DV_launch) + self._kv_custom_scratch(), head_dim=self.D,
                             head_dim_v=self.DV_launch, elem_bytes=2, n_rowscales=self.n_rowscales,
                             mask_mode=mask_mode, table_rows=table_rows if mask_mode == 2 else 0)
            v = self._variants[key] = (module, cfg, cfg_src)
        return v

    # ---- launch ----------------------------------------------------------------------------
    def __call__(self, q, k, v, *extra):
        """Forward; records the autograd edge when a gradient of q, k or v is wanted (the reference's
        generated ``_attention`` autograd function, attn_tl.py:530-640)."""
        if torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in (q, k, v)):
            return _PrefillFunction.apply(self, q, k, v, *extra)
        return self._forward(q, k, v, *extra)

    def backward_op(self):
        if getattr(self, "_bwd", None) is None:
            from .prefill_bwd_op import PrefillBwdOp
            self._bwd = PrefillBwdOp(self, *self._graph, tune=self._tune_bwd[0], tune_file=self._tune_bwd[1],
                                     allow_spills=self.allow_spills)
        return self._bwd

    def _forward(self, q, k, v, *extra):
        try:
            return self._forward_once(q, k, v, *extra)
        except rt.SpillError:
            # (raised by the compilation of a variant, before anything was launched)
            if not self._gives_way_to_the_generic_kernel():
                raise
            return self._forward_once(q, k, v, *extra)

    def _forward_once(self, q, k, v, *extra):
        if self._tune_pending:
            self._tune(q, k, v, *extra)
        n_custom = len(self.functors.customs)
        extern_mask = None
        if len(extra) == n_custom + 1:
            extern_mask = extra[-1]
            extra = extra[:-1]
        if len(extra) != n_custom:
            raise TypeError(f"expected {n_custom} custom input tensor(s), got {len(extra)}")
        for name, t in (("q", q), ("k", k), ("v", v)):
            if not (isinstance(t, torch.Tensor) and t.is_cuda):
                raise RuntimeError(f"{name} must be a tensor on the GPU (there is no CPU path)")
            if t.dtype != self.dtype:
                raise TypeError(f"{name} has dtype {t.dtype}, the engine was built for {self.dtype}")
            if t.dim() != 4:
                raise ValueError(f"{name} must be [batch, seq, heads, dim]")
        B, Sq, Hq, D = q.shape
        Bk, Skv, Hkv, Dk = k.shape
        if (D, Dk, v.shape[3]) != (self.D, self.D, self.DV):
            raise ValueError(f"head dims {(D, Dk, v.shape[3])} differ from the compiled {(self.D, self.D, self.DV)}")
        if Bk != B or v.shape[0] != B or v.shape[1] != Skv or v.shape[2] != Hkv or Hq % Hkv:
            raise ValueError("inconsistent q/k/v shapes")
        q, k, v = (rt.rows_for_kernels(t) for t in (q, k, v))
        dev = q.device

        if extern_mask is not None and extern_mask is self.block_mask and not self.extern_block_mask:
            # the block mask this engine inferred from mask_mod itself (AttentionEngine appends it to every
            # call, attn_engine.py:391-392 of the reference): the tile-class table planned from the same
            # mask_mod says the same at the kernel's own tile granularity, whatever infer_mask_block_M/N are
            extern_mask = None
        if extern_mask is not None:
            bm, bn = self.mask_block
            if bn % self.tiles.block_n or (self.tiles.block_m % bm and bm % self.tiles.block_m) or \
                    self.tiles.block_m > self.MASK_ROWS_PER_TILE * bm:
                raise NotImplementedError(
                    f"a block mask of {bm}x{bn} blocks does not fit the kernel's {self.tiles.block_m}x"
                    f"{self.tiles.block_n} tiles (construct the engine with extern_block_mask=True)")
            table = extern_mask
            if table.dim() != 4:
                raise ValueError("block_mask must be [B|1, H|1, Sq/bm, Skv/bn]")
            if table.dtype != torch.int8:
                table = table.to(torch.int8)
            table = table.to(dev).contiguous()
            mode, mbm, mbn = 2, bm, bn
        else:
            plan = self._plan(B, Hq, Sq, Skv, dev)
            mode, table, mbm, mbn = plan.mode, plan.table, plan.block_m, plan.block_n
        n_split, kv_per_split = self.plan_splits(B, Hq, Sq, Skv)
        module, cfg, _ = self._variant(mode, Sq % self.tiles.block_m == 0, Skv % self.tiles.block_n == 0, n_split,
                                       self._table_rows(mbm) if mode == 2 else 1,
                                       extern_mask is None and plan.heavy_last)
        kern = module.kernel("ae_prefill_kernel")

        out = torch.empty((B, Sq, Hq, self.DV), dtype=self.dtype, device=dev)
        rowscales = [torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev) for _ in range(self.n_rowscales)]
        p = rt.AttnParams()
        p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
        p.q_stride_b, p.q_stride_s, p.q_stride_h, _ = q.stride()
        p.k_stride_b, p.k_stride_s, p.k_stride_h, _ = k.stride()
        p.v_stride_b, p.v_stride_s, p.v_stride_h, _ = v.stride()
        p.o_stride_b, p.o_stride_s, p.o_stride_h, _ = out.stride()
        p.batch, p.heads_q, p.heads_kv, p.seqlen_q, p.seqlen_kv = B, Hq, Hkv, Sq, Skv
        for i, r in enumerate(rowscales):
            p.rowscale_out[i] = r.data_ptr()
        keep = []
        for i, (desc, t) in enumerate(zip(self.functors.customs, extra)):
            t = t.to(device=dev, dtype=desc.torch_dtype).contiguous()
            keep.append(t)
            p.custom[i] = t.data_ptr()
        if mode == 2:
            p.block_mask = table.data_ptr()
            p.mask_b, p.mask_h, p.mask_nq, p.mask_nkv = table.shape
            p.mask_block_m, p.mask_block_n = mbm, mbn
            keep.append(table)
        stream = rt.current_stream(dev)
        if n_split > 1:
            partial_o = torch.empty((B, Sq, Hq, n_split, self.DV), dtype=torch.float32, device=dev)
            partial_rs = torch.empty((max(1, self.n_rowscales), B, Sq, Hq, n_split), dtype=torch.float32, device=dev)
            p.partial_o, p.partial_rs = partial_o.data_ptr(), partial_rs.data_ptr()
            p.num_splits, p.kv_per_split = n_split, kv_per_split
            keep += [partial_o, partial_rs]
            ccfg = rt.TileCfg(block_m=1, block_n=n_split, threads=self.COMBINE_THREADS, lds_bytes=0,
                              head_dim=self.D, head_dim_v=self.DV, elem_bytes=2,
                              n_rowscales=self.n_rowscales, mask_mode=0)
            rt.prefill_split_fwd(kern, module.kernel("ae_decode_combine_kernel"), p, cfg, ccfg, stream)
        else:
            if self._clock_stamps():
                n_wg = -(-Sq // self.tiles.block_m) * (-(-(B * Hq) // 8) * 8)
                self.clock_stamps = torch.zeros((n_wg, 2), dtype=torch.int64, device=dev)
                p.partial_o = self.clock_stamps.data_ptr()
            # one launch per slice of DV_launch value columns (a single one unless DV > 256)
            esz = v.element_size()
            for c0 in range(0, self.DV, self.DV_launch):
                p.v = v.data_ptr() + c0 * esz
                p.out = out.data_ptr() + c0 * esz
                rt.prefill_fwd(kern, p, cfg, stream)
        self.final_rowscales = dict(zip(self.functors.final_rowscale_names, rowscales))
        self._keepalive = keep
        return out


class _PrefillFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, op, q, k, v, *extra):
        # `extra`: the block mask the engine inferred from mask_mod, which it appends to every call (the
        # backward applies mask_mod per element instead); custom inputs and external masks are refused.
        # A graph without a backward still runs forward on tensors that require gradients -- a caller who
        # only wants `out` from leaf tensors gets it -- and says so when .backward() is called, as the
        # reference does (its generated _attention.backward is where a missing rule surfaces,
        # attn_tl.py:582-640).
        try:
            bwd, ctx.no_backward = op.backward_op(), None
        except NotImplementedError as e:
            bwd, ctx.no_backward = None, e
        with torch.no_grad():
            out = op._forward(q.detach(), k.detach(), v.detach(), *extra)
        ctx.op = op
        ctx.n_extra = len(extra)
        if bwd is None:
            return out
        ctx.customs = tuple(extra[:len(op.functors.customs)])       # scalar CustomIO tensors of score_mod
        # the user's block mask of this call (engines built with extern_block_mask=True): last positional
        ctx.block_mask = extra[-1] if (op.extern_block_mask and len(extra) == len(op.functors.customs) + 1) else None
        # the final row scales the backward reads: lse, or every final row scale of an online function whose
        # forward() / backward() are traced
        scales = [op.final_rowscales[n] for n in bwd.rowscale_names] or [q.new_empty(0)]
        ctx.save_for_backward(q, k, v, out, *scales)
        return out

    @staticmethod
    def backward(ctx, dout):
        if ctx.no_backward is not None:
            raise NotImplementedError(str(ctx.no_backward)) from ctx.no_backward
        q, k, v, out, *scales = ctx.saved_tensors
        lse = scales[0] if len(scales) == 1 else scales
        dq, dk, dv = ctx.op.backward_op()(q, k, v, out, lse, dout, ctx.customs, ctx.block_mask)
        return (None, dq, dk, dv) + (None,) * ctx.n_extra
