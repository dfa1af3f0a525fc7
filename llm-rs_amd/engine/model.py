"""A model as data: token table, blocks built from a `ModelSpec`, the order they
run in, final norm and output matrix.  It knows no architecture; the typed
configuration's `model_spec()` does (config/llama.py).  Reference counterpart:
LlamaModel / run_layers (src/arch/llama.rs:24-43, :146-172)."""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional, Tuple

import torch

from ..config.spec import ModelSpec
from ..kernels import EPI_STORE_F32, kernels
from ..parts import TensorSpec, build_block, build_norm, place
from ..weights import check_tensors


class Model:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        spec.validate()
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine computes in float32 or bfloat16, not {dtype}")
        self.spec, self.dtype, self.device = spec, dtype, torch.device(device)
        self.blocks = [build_block(layer, dtype) for layer in spec.layers]
        self.final_norm = build_norm(spec.final_norm, dtype) if spec.final_norm is not None else None
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        keyed = {}
        for block in self.blocks:
            for part in block.parts():
                if part.recording_signature is not None:
                    keyed.setdefault(part.recording_signature, part)
        self._keyed_parts = list(keyed.values())

    # -- weights -------------------------------------------------------------
    def tensors(self) -> Dict[str, TensorSpec]:
        s = self.spec
        out = {s.embedding_name: TensorSpec((s.vocab_size, s.hidden_size))}
        if s.head_name is not None:
            out[s.head_name] = TensorSpec((s.vocab_size, s.hidden_size))
        for block in self.blocks:
            for part in block.parts():
                out.update(part.tensors())
        if self.final_norm is not None:
            out.update(self.final_norm.tensors())
        return out

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Takes every tensor `tensors()` names; anything missing, left over or
        of another shape is reported in one error."""
        want = {n: t.shape for n, t in self.tensors().items()}
        # (a mapping that makes or reads its tensors only when asked says their shapes without doing so)
        have = tensors.shapes() if hasattr(tensors, "shapes") else {n: tuple(t.shape) for n, t in tensors.items()}
        check_tensors(have, want, ignorable=self.spec.ignorable_tensors)
        s = self.spec
        self.embedding = place(tensors[s.embedding_name], self.device, self.dtype)
        # tied: the output matrix is the token table (src/arch/llama.rs:81)
        self.head = self.embedding if s.head_name is None else place(tensors[s.head_name], self.device, self.dtype)
        for block in self.blocks:
            for part in block.parts():
                part.load(tensors, self.device)
        if self.final_norm is not None:
            self.final_norm.load(tensors, self.device)

    def weights(self) -> Dict[str, torch.Tensor]:
        """Every tensor of the model on the host, under its file name and in the file's layout
        (what parts fused or reordered at load is undone), in the dtype the engine keeps it in:
        what `load` would take again, and what another implementation can be given to compare."""
        s = self.spec
        out = {s.embedding_name: self.embedding.cpu()}
        if s.head_name is not None:
            out[s.head_name] = self.head.cpu()
        for block in self.blocks:
            for part in block.parts():
                out.update(part.export())
        if self.final_norm is not None:
            out.update(self.final_norm.export())
        return out

    def weight_bytes_per_step(self) -> int:
        """Bytes of weights one step reads when it uses each once (the table's rows aside):
        every tensor a part of the schedule's layers holds, the final norm's, and the output matrix."""
        seen = set()
        total = sum(part.step_weight_bytes(seen) for run in self.spec.schedule for part in self.blocks[run.layer].parts())
        if self.final_norm is not None:
            total += self.final_norm.step_weight_bytes(seen)
        if self.head.data_ptr() not in seen:
            total += self.head.numel() * self.head.element_size()
        return total

    def graph_safe(self) -> bool:
        """Whether a step of this model may be recorded into a HIP graph (every part says so)."""
        return (all(part.graph_safe for block in self.blocks for part in block.parts())
                and (self.final_norm is None or self.final_norm.graph_safe))

    def recording_key(self, ctx) -> tuple:
        """What a recording of this step depends on beyond its sizes (its parts say)."""
        return tuple(part.recording_key(ctx) for part in self._keyed_parts)

    # -- cache ---------------------------------------------------------------
    def cache_needs(self) -> List[Tuple[object, Optional[int]]]:
        return [(self.blocks[run.layer].cache_need(), run.cache_of) for run in self.spec.schedule]

    # -- one step --------------------------------------------------------------
    def forward(self, ctx, cache_views) -> Optional[torch.Tensor]:
        """Runs the step's T tokens through the schedule; returns float32 logits
        [n_want, vocab] at the wanted rows, or None when none is wanted."""
        k = kernels()
        T = ctx.n_tokens
        h = ctx.workspace("model.h", (T, self.spec.hidden_size), torch.float32)
        k.embed_rows(h, self.embedding, ctx.tokens, self.spec.embedding_scale)
        ctx.note_left(h, None)
        for i, run in enumerate(self.spec.schedule):
            ctx.run_index = i
            block = self.blocks[run.layer]
            # the norm that reads the stream after this block: the next block's first; after the last block the
            # final norm, where it reads every row (else it reads gathered rows and runs as a kernel of its own)
            later = self.spec.schedule[i + 1] if i + 1 < len(self.spec.schedule) else None
            ctx.norm_after_block = (self.blocks[later.layer].first_norm() if later is not None
                                    else self.final_norm if ctx.wants_every_row else None)      # (None too without a final norm)
            block.forward(ctx, h, cache_views[i])
            if not block.keeps_left_current:
                ctx.note_left(h, None)
        ctx.norm_after_block = ctx.upcoming_norm = None
        if ctx.n_want == 0:
            return None
        # Norm only the wanted rows, then the output matrix: the reference norms all
        # rows and gathers after (src/arch/llama.rs:135-139), which is the same numbers.
        # (A step of few single tokens that wants them all: the last product has prepared the final norm, and the
        # output matrix's product finishes it; no norm kernel runs.)
        x = self.final_norm.deferred(ctx, h) if ctx.wants_every_row and self.final_norm is not None else None
        if x is None:
            x = ctx.workspace("model.head_in", (ctx.n_want, self.spec.hidden_size), self.dtype)
            if self.final_norm is not None:
                self.final_norm.forward(ctx, h, x, ctx.want_rows)
            else:       # no norm before the output matrix: the wanted rows of the stream, in the activation type
                rows = x if self.dtype == torch.float32 else ctx.workspace("model.head_rows", x.shape, torch.float32)
                k.embed_rows(rows, h, ctx.want_rows, 1.0)
                if rows is not x:
                    k.cast(x, rows)
        logits = ctx.workspace("model.logits", (ctx.n_want, self.spec.vocab_size), torch.float32)
        k.gemm(x, self.head, logits, EPI_STORE_F32, ctx.gemm_workspace(x, self.head))
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap > 0.0:
            k.scale_softcap_rows(logits, self.spec.logit_scale, self.spec.logit_softcap)
        return logits
