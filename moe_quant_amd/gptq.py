"""Drop-in for MoE-Quant's src/gptq.py: the same `GPTQ` handle, its numeric work done by HIP kernels.

Out of scope (raise instead of silently differing): asymmetric grids, conv layers, the multi-GPU
Hessian all-reduce.  `update` takes bf16, fp16 or fp32 activations, the dtypes the reference's driver
offers (quant.py:79-81): 16-bit tokens are read as they are by the matrix cores (their pairwise
products are exact in fp32, so nothing is lost versus the reference's up-cast, src/gptq.py:97), fp32
tokens go through fp32-accurate GEMM tiles.  `quantization_scale="mse"` runs the scale search."""
from __future__ import annotations

import warnings
from enum import Enum
from typing import Optional, Tuple

import numpy as np
import torch
import torch.nn as nn
from torch import Tensor

from . import linalg_utils, ops


_ACT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


class QuantizationOrder(Enum):
    DEFAULT = "default"
    ACTIVATION = "activation"


class GPTQ:
    """Mirror of src/gptq.py:22-243 (constructor arguments, attributes and methods keep their names)."""

    # factorisations computed so far by all handles (a tied handle that reuses its owner's adds none); a plain class
    # counter for tests and logs, not synchronised between host threads
    factor_calls = 0

    def __init__(
        self,
        layer: nn.Module,
        group_size: Optional[int] = None,
        sym: bool = False,
        rel_damp: float = 1e-2,
        block_size: int = None,
        quantization_order: str = "default",
        quantization_scale: str = "absmax",
        is_distributed: bool = False,
        tied_gptq_handle: Optional["GPTQ"] = None,
    ):
        self._validate_layer(layer)
        self.layer = layer
        self._W = self.layer.weight
        self._W_lazy = False
        self.d_row, self.d_col = layer.weight.shape[0], int(np.prod(layer.weight.shape[1:]))  # src/model_utils.py:11-12
        self.sym = sym
        self.group_size = group_size
        self.rel_damp = rel_damp
        self.block_size = block_size or self.d_col
        self.quantization_order = QuantizationOrder(quantization_order)
        # "absmax" or "mse".  The reference compares this string with an Enum member (src/quant_utils.py:221),
        # which never matches, so its scale search is dead code; here "mse" runs the search.
        if quantization_scale not in ("absmax", "mse"):
            raise ValueError(f"quantization_scale must be 'absmax' or 'mse', got {quantization_scale!r}")
        self.quantization_scale = quantization_scale
        self.W_device = self.W.device
        self.W_dtype = self.W.dtype
        self.W_shape = self.W.shape
        self.H = None
        self.num_samples = 0
        self.is_distributed = is_distributed
        self.tied_gptq_handle = tied_gptq_handle
        self.num_tied_handles = 0
        if tied_gptq_handle is not None:
            tied_gptq_handle.num_tied_handles += 1
        self.issue_zero_samples = False
        self._issue_nan_hessian = False
        self._issue_non_invertible = False
        # device-side verdicts of the last pre-step / factorisation; read back only when somebody asks
        self._flags = None
        self._flags_unread = False
        self._info = None
        self._pruned = None
        self._H_upper_only = False  # H holds only its upper triangle (state of the handle that owns H)
        self._H_clean = False  # H went through the pre-step scan and nothing touched it since (idem)
        # engine state shared with tied handles (the reference recomputes both for every tied handle)
        self._perm = None
        self._hessian_inv = None  # U, when somebody asked for it through _get_hessian_inverse
        self._loop_factor = None  # F, the multipliers the quantize path hands to the loop (kept for tied handles)

    # The reference keeps three host booleans and pays a device->host read for two of them inside quantize().
    # Here the verdicts stay on the device (so linears can be queued back to back on several streams) and are
    # fetched when one of these attributes is read.
    @property
    def issue_nan_hessian(self) -> bool:
        if self._flags_unread and self._flags is not None:
            self._issue_nan_hessian = self._issue_nan_hessian or bool(self._flags[0].item())
            self._flags_unread = False
        return self._issue_nan_hessian

    @issue_nan_hessian.setter
    def issue_nan_hessian(self, v: bool) -> None:
        self._issue_nan_hessian, self._flags_unread = bool(v), False

    @property
    def issue_non_invertible(self) -> bool:
        if self._info is not None:
            self._issue_non_invertible = self._issue_non_invertible or int(self._info.item()) != 0
            self._info = None
        return self._issue_non_invertible

    @issue_non_invertible.setter
    def issue_non_invertible(self, v: bool) -> None:
        self._issue_non_invertible, self._info = bool(v), None

    @property
    def W(self) -> Tensor:
        """`layer.weight` before the pre-step; afterwards the fp32 copy with pruned input channels zeroed that
        the reference keeps (src/gptq.py:148-152), materialised on first use: the kernels read the layer's own
        weights plus the pruned mask instead."""
        if self._W_lazy:
            w = self.layer.weight.detach().clone().float()
            if self._pruned is not None:
                w = torch.where(self._pruned.bool()[None, :], torch.zeros((), device=w.device), w)
            self._W, self._W_lazy = w, False
        return self._W

    @W.setter
    def W(self, w: Tensor) -> None:
        self._W, self._W_lazy = w, False

    @staticmethod
    def _validate_layer(layer):
        assert isinstance(layer, nn.Linear), "this engine supports nn.Linear layers only"

    def has_hessian_issues(self) -> bool:
        return any([self.issue_zero_samples, self.issue_nan_hessian, self.issue_non_invertible])

    # ---- Hessian accumulation: src/gptq.py:73-105 ---------------------------------------------------
    @torch.no_grad()
    def update(self, input) -> None:
        """`input`: the activations the forward hook delivers (..., C), or an `ops.PackedTokens` of them (the same
        tokens in the layout the matrix cores read, for callers that copy the tokens anyway: ops.pack_tokens gathers
        and re-lays them out in one pass, ops.swiglu_packed writes a down projection's inputs that way)."""
        if isinstance(input, ops.PackedTokens):
            return GPTQ.update_many([self], [input])
        input = input.reshape(-1, input.shape[-1])
        if input.dtype not in _ACT_DTYPES:
            raise TypeError(f"GPTQ.update takes bf16, fp16 or fp32 activations, got {input.dtype}")
        num_new_samples = input.shape[0]
        if num_new_samples == 0:
            # Nothing to add (an expert that received no token in this batch).  With samples collected before,
            # the reference's update is the identity (beta = 1, alpha * 0); with none it divides 0/0.  Either way
            # H is left as it is: a handle that never sees a token keeps H = None and takes the pre-step's
            # identity / issue_zero_samples path, exactly like a handle whose hook never fired.
            return
        if self.H is None:
            # the first product runs with beta = 0 and writes the whole upper triangle, the pre-step mirrors it:
            # no need to clear 4*C^2 bytes first
            alloc = torch.empty if self.num_samples == 0 else torch.zeros
            self.H = alloc((self.d_col, self.d_col), device=input.device, dtype=torch.float32)
        beta = self.num_samples / (self.num_samples + num_new_samples)
        alpha = 2.0 / (self.num_samples + num_new_samples)
        # only the upper triangle is accumulated; quantization_pre_step mirrors it once
        ops.hessian_syrk_(self.H, input, beta, alpha, mirror=False)
        self._H_upper_only = True
        self._H_clean = False
        self.num_samples += num_new_samples

    add_batch = update

    @staticmethod
    @torch.no_grad()
    def update_many(handles, inputs) -> None:
        """`h.update(x)` for several handles of one input width with one library call (the experts of a block,
        whose hooks the reference serves one addmm_ at a time).  Same arithmetic per handle as `update`."""
        Hs, Xs, betas, alphas = [], [], [], []
        inputs = list(inputs)
        packed = bool(inputs) and isinstance(inputs[0], ops.PackedTokens)
        if any(isinstance(x, ops.PackedTokens) != packed for x in inputs):
            raise TypeError("update_many takes either tensors or PackedTokens, not a mix")
        for h, x in zip(handles, inputs):
            if packed:
                if x.C != h.d_col:
                    raise ValueError(f"packed tokens have {x.C} channels, the layer {h.d_col}")
                n_x = x.n
            else:
                x = x.reshape(-1, x.shape[-1])
                if x.dtype not in _ACT_DTYPES:
                    raise TypeError(f"GPTQ.update takes bf16, fp16 or fp32 activations, got {x.dtype}")
                n_x = x.shape[0]
            if n_x == 0:
                continue
            if h.H is None:
                alloc = torch.empty if h.num_samples == 0 else torch.zeros  # beta = 0 below: nothing to clear
                h.H = alloc((h.d_col, h.d_col), device=(x.data if packed else x).device, dtype=torch.float32)
            n = n_x
            Hs.append(h.H)
            Xs.append(x)
            betas.append(h.num_samples / (h.num_samples + n))
            alphas.append(2.0 / (h.num_samples + n))
            h.num_samples += n
            h._H_upper_only, h._H_clean = True, False
        if packed:
            if len(Hs) == 1:
                ops.hessian_syrk_packed_(Hs[0], Xs[0], betas[0], alphas[0], mirror=False)
            else:
                ops.hessian_syrk_packed_grouped_(Hs, Xs, betas, alphas, mirror=False)
        else:
            ops.hessian_syrk_grouped_(Hs, Xs, betas, alphas, mirror=False)

    @property
    def tokens_collected(self) -> int:
        return self.num_samples

    def reset(self) -> None:
        """src/gptq.py:111-120."""
        self.W = self.layer.weight
        if self.num_tied_handles == 0:
            self.H = None
            self._hessian_inv = self._loop_factor = None
            self._H_upper_only = self._H_clean = False
            self._perm = None
        elif self.tied_gptq_handle:
            self.tied_gptq_handle.num_tied_handles -= 1
            if self.tied_gptq_handle.num_tied_handles == 0:
                self.tied_gptq_handle.H = None
                self.tied_gptq_handle._hessian_inv = self.tied_gptq_handle._loop_factor = None
                self.tied_gptq_handle._H_upper_only = self.tied_gptq_handle._H_clean = False
                self.tied_gptq_handle._perm = None
        # (while tied handles still need this handle's H -- permuted in place under act-order -- the column order that
        # goes with it is kept as well, like H and the factor: whether the owner is reset before its tied handles are
        # quantized, as the reference's driver does (quant.py:297-330), or after, they pair permuted weights with the
        # permuted H.  The reference re-sorts the already sorted diagonal there and pairs un-permuted weights with it.)
        self.num_samples = 0
        if self.tied_gptq_handle is not None:
            self._perm = None
        self._pruned = None
        if self.tied_gptq_handle is not None:
            self._hessian_inv = self._loop_factor = None
        torch.cuda.empty_cache()

    # ---- pre-step: src/gptq.py:122-154 --------------------------------------------------------------
    def _hessian_owner(self) -> "GPTQ":
        t = self.tied_gptq_handle
        return t if (t is not None and self.H is t.H) else self

    def symmetrize_hessian(self) -> None:
        """`update` maintains the upper triangle of H only; this mirrors it onto the lower one."""
        owner = self._hessian_owner()
        if self.H is not None and owner._H_upper_only:
            ops.symmetrize_upper_(self.H)
            owner._H_upper_only = False

    @torch.no_grad()
    def quantization_pre_step(self) -> None:
        if self.H is None:
            if self.tied_gptq_handle:
                self.H = self.tied_gptq_handle.H
            else:
                self.H = torch.eye(self.d_col, device=self.W_device, dtype=torch.float32)
                self.issue_zero_samples = True
        if self.H is None:  # tied to a handle that holds no Hessian either
            self.H = torch.eye(self.d_col, device=self.W_device, dtype=torch.float32)
            self.issue_zero_samples = True
        if self.is_distributed and torch.distributed.is_available() and torch.distributed.is_initialized():
            if torch.distributed.get_world_size() > 1:
                raise NotImplementedError("the multi-GPU Hessian all-reduce is outside this engine's scope")
        owner = self._hessian_owner()
        if owner is not self and owner._H_clean:
            # the owner's pre-step already scanned (and its quantize damped) this very matrix: no NaN, no zero
            # on the diagonal is left to find (the reference scans it again for every tied handle)
            self._pruned, self._flags, self._flags_unread = None, None, False
        else:
            # NaN -> identity, zero diagonal -> 1 (+ the mirror of the upper triangle), all on the device
            self._pruned, self._flags = ops.hessian_prestep_(self.H, owner._H_upper_only)
            self._flags_unread = True
            owner._H_upper_only = False
            owner._H_clean = True
        self._W, self._W_lazy = None, True
        self.pre_step_completed = True

    # ---- quantize: src/gptq.py:156-218 ---------------------------------------------------------------
    @torch.no_grad()
    def _prepare(self, bits: int) -> dict:
        """Everything `_quantize` does before the factorisation: scales from the un-updated weights, the column
        order, H permuted in place of the reference's `H[perm][:, perm]`."""
        if not self.sym:
            raise NotImplementedError("only symmetric quantization is supported (as MoE-Quant's README states)")
        d_col, dtype, device = self.d_col, self.W_dtype, self.W_device
        group_size = self.group_size or d_col
        W, dead = self._kernel_weights()
        # per-group scales from the un-updated weights (src/gptq.py:171-178): compact (R,G) and (G,R)
        scale_rg, scale_gr = ops.quant_grid_sym(W, group_size, bits, dtype, dead_cols=dead)
        if self.quantization_scale == "mse":  # src/quant_utils.py:221-232 with its default search grid
            points = torch.linspace(1, 0.2, 100, dtype=torch.float32, device=device)
            ops.mse_scale_sym_(W, group_size, points, scale_rg, scale_gr, float(2 ** (bits - 1)), float(2**bits - 1), 2.4,
                               dtype, dead_cols=dead)
        tied = self.tied_gptq_handle
        perm = perm_i32 = perm_inv_i32 = None
        if self.quantization_order == QuantizationOrder.ACTIVATION:
            if tied is not None and tied._perm is not None:
                # the owner's H is already permuted; reuse its order (the reference re-sorts the sorted
                # diagonal here, gets the identity and pairs un-permuted weights with a permuted H)
                perm = tied._perm
            else:
                perm = torch.argsort(self.H.diag(), descending=True)
            perm_inv = torch.argsort(perm)
            perm_i32, perm_inv_i32 = perm.to(torch.int32), perm_inv.to(torch.int32)
            self._perm = perm
            if tied is None:
                self.H = ops.permute_symmetric(self.H, perm_i32)  # src/gptq.py:187, one pass, no second temporary
        if perm is None:
            scale_row = torch.arange(d_col, device=device, dtype=torch.int32) // group_size
        else:
            scale_row = (perm // group_size).to(torch.int32)
        return dict(W=W, dead=dead, scale_rg=scale_rg, scale_gr=scale_gr, perm_i32=perm_i32, perm_inv_i32=perm_inv_i32,
                    scale_row=scale_row, maxq=float(2**bits - 1), qzero=float(2 ** (bits - 1)))

    def _finish(self, ctx: dict, Qt: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
        """The reference's post-loop casts (src/gptq.py:199-202)."""
        self._Qt, self._perm_inv_i32 = Qt, ctx["perm_inv_i32"]
        qweight = ops.untranspose_codes(Qt, ctx["perm_inv_i32"])
        scale = ctx["scale_rg"].to(self.W_dtype)
        zero = torch.full_like(scale, ctx["qzero"])
        return qweight, scale, zero

    @torch.no_grad()
    def _quantize(self, bits: int) -> Tuple[Tensor, Tensor, Tensor]:
        return GPTQ._quantize_prepared([self], [self._prepare(bits)])[0]

    @staticmethod
    def _quantize_prepared(handles, ctxs):
        """Factorisation, column loop and post-loop casts for handles of one shape whose `_prepare` has run.

        The loop runs in its inverse-free form: with H = R R^T (R upper), the reference's factor is U = R^-1
        (src/gptq.py:236-242) and its recurrence x_k = w_k + sum_{j<k} e_j U[j,k]/U[j,j] equals
        x_k = w_k - (1/R_kk) sum_{j<k} z_j R[j,k] with z_j the total change of column j, so only the Cholesky factor
        is computed (half the flop) and the loop gets F = -R[j,k]/R[k,k] and a copy of the original weights.
        `_get_hessian_inverse` / `gptq_loop.gptq_loop` keep the reference's U-based forms."""
        h0 = handles[0]
        # factors: reuse what tied owners hold, factor the rest side by side
        need = []
        for h in handles:
            tied = h.tied_gptq_handle
            shares = tied is not None and tied.H is h.H
            if shares and (tied._loop_factor is not None or any(tied is o for o in need)):
                continue  # the owner's factor: already there, or computed below
            h._damp_hessian()
            need.append(h)
        own = {}
        if need:
            Hs = [o.H for o in need]
            C = h0.d_col
            if C % 128 or any(H.dtype != torch.float32 or H.stride(1) != 1 or H.stride(0) != C or H.data_ptr() % 16
                              for H in Hs):
                Hs = [linalg_utils._padded_copy(H) for H in Hs]  # identity-padded to a multiple of 128, contiguous
            Fs, infos = ops.factor_chol_grouped(Hs)
            GPTQ.factor_calls += len(need)
            for i, o in enumerate(need):
                own[id(o)], o._info = Fs[i], infos[i:i + 1]
                if o.num_tied_handles > 0:
                    o._loop_factor = Fs[i]
        Fs = []
        for h in handles:
            tied = h.tied_gptq_handle
            Fs.append(own[id(h)] if id(h) in own else (own[id(tied)] if id(tied) in own else tied._loop_factor))
        pairs = [ops.prepare_wt_pair(c["W"], c["perm_i32"], dead_cols=c["dead"]) for c in ctxs]
        Qts = ops.gptq_loop_chol_grouped_([p[0] for p in pairs], [p[1] for p in pairs], Fs, [c["scale_gr"] for c in ctxs],
                                          [c["scale_row"] for c in ctxs], ctxs[0]["qzero"], ctxs[0]["maxq"], h0.W_dtype,
                                          h0.block_size)
        return [h._finish(c, Qt) for h, c, Qt in zip(handles, ctxs, Qts)]

    @staticmethod
    @torch.no_grad()
    def quantize_many(handles, bits: int):
        """`[h.quantize(bits) for h in handles]` for linears of one shape and one configuration (the experts of a
        block, which the reference quantizes one after another, quant.py:291-386), with the two long phases --
        factorisation and column loop -- run as one grouped library call each: a lone factorisation or loop is a
        chain of dependent launches that cannot fill the GPU.  Same results, bit for bit, as one call per handle,
        with or without a `reset()` of the owner between the calls.
        A tied handle must come after its owner (in this list or in an earlier call)."""
        handles = list(handles)
        if not handles:
            return []
        h0 = handles[0]
        key = lambda h: (h.d_row, h.d_col, h.W_dtype, h.group_size, min(h.block_size, 128), h.sym, h.W_device)
        if any(key(h) != key(h0) for h in handles):
            raise ValueError("quantize_many needs linears of one shape, dtype, group size and block size")
        ctxs = []
        for h in handles:  # in list order: a tied handle picks up what its owner's steps left (H, column order)
            h.quantization_pre_step()
            h._pin_inputs_to_current_stream()
            ctxs.append(h._prepare(bits))
        return GPTQ._quantize_prepared(handles, ctxs)

    def _kernel_weights(self):
        """(weights, pruned mask) the kernels read: after the pre-step the layer's own weights plus the mask stand
        for the reference's fp32 copy with zeroed columns, unless somebody has touched or replaced that copy."""
        if self._W_lazy:
            return self.layer.weight.detach(), self._pruned
        return self._W.detach(), None

    def quantize(self, bits: int | float) -> Tuple[Tensor, Tensor, Tensor]:
        self.quantization_pre_step()
        self._pin_inputs_to_current_stream()
        return self._quantize(bits)

    def _pin_inputs_to_current_stream(self) -> None:
        """The layer's weight and H were allocated on whatever stream loaded the model / ran the hooks; a caller may
        run `quantize` on another stream and drop its last reference to either (`layer.weight.data = ...`,
        `handle.H = None`) while this stream's kernels are still queued.  Telling the caching allocator that this
        stream uses them keeps it from handing their memory to a new tensor before those kernels have run."""
        if not self.W_device.type == "cuda":
            return
        cur = torch.cuda.current_stream(self.W_device)
        for t in (self.layer.weight, self.H):
            if isinstance(t, Tensor) and t.is_cuda:
                t.record_stream(cur)

    def packed_words(self) -> Tensor:
        """int32 (R, C/8) compressed_tensors words of the last `quantize` call, packed straight from the
        loop's own code buffer (same bits as pack_weight on the returned qweight)."""
        return ops.pack_from_qt(self._Qt, self._perm_inv_i32)

    # ---- inverse factor: src/gptq.py:220-243 ---------------------------------------------------------
    def _damp_hessian(self) -> None:
        """All-zero weight columns -> unit rows/columns of H, then damping (src/gptq.py:221-234); a tied handle finds
        both done by its owner."""
        if not self.tied_gptq_handle:
            H = self.H
            flags = self._flags if self._flags is not None else torch.zeros(4, dtype=torch.int32, device=H.device)
            w, pruned = self._kernel_weights()
            ops.hessian_damp_(H, w, pruned, self.rel_damp, flags)
            self._H_clean = True

    def _factor_hessian(self) -> Tensor:
        # a failed factorisation yields the identity on the device, the reference's `except` branch
        # (src/gptq.py:239-240, which never sets issue_non_invertible; this engine does)
        U, self._info = linalg_utils.inverse_cholesky_factor(self.H)
        GPTQ.factor_calls += 1
        if self.num_tied_handles > 0:
            self._hessian_inv = U
        return U

    @torch.no_grad()
    def _get_hessian_inverse(self) -> Tensor:
        tied = self.tied_gptq_handle
        if tied is not None and tied._hessian_inv is not None and tied.H is self.H:
            return tied._hessian_inv  # same damped H -> same factor; the reference recomputes it
        self._damp_hessian()
        return self._factor_hessian()
