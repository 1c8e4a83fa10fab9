"""Stage inputs: where the rows of a stage come from."""
from __future__ import annotations

from .base import STAGE_INPUTS, build_part, to_compute
from .spec import StateNeed


@STAGE_INPUTS.register("token_embedding")
class TokenEmbedding:
    """x = E[token] (reference main_models_new.py:199)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {}

    @classmethod
    def state_need(cls, params):
        return None

    def __init__(self, spec, tensors, ops):
        self.ops = ops

    def forward(self, batch, previous, shared, state):
        return self.ops.embedding(shared["embedding"], batch.tokens)


@STAGE_INPUTS.register("fuse_previous_stage")
class FusePreviousStage:
    """x = [h ; norm_e(E[token])] . Wp, h being the previous stage's output at the same position.

    The previous stage's output is already normed; only the embedding gets a norm of its own (reference
    main_models_new.py:163-164). A stage of lag j runs at the positions [s-j, e-j) when the step brings the
    tokens of positions [s, e); the previous stage ran [s-j+1, e-j+1). So the hidden row of position s-j
    was made one step earlier and waits in this part's per-request state (one row of d_model), and the
    previous stage's last row of this step, position e-j, is kept there for the next step.

    params: d_model, embed_norm (a PartSpec). tensors: proj (2*d_model, d_model), stored [in, out].
    """
    graph_safe = True
    reads_previous = True

    @classmethod
    def tensor_shapes(cls, params):
        d = params["d_model"]
        shapes = {"proj": (2 * d, d)}
        return shapes

    @classmethod
    def state_need(cls, params):
        return StateNeed((params["d_model"],), "compute")

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.d_model = int(spec.params["d_model"])
        self.w_proj = to_compute(ops, tensors.of(spec, "proj").t())          # [d_model, 2*d_model]
        self.embed_norm = build_part(spec.params["embed_norm"], tensors, ops)

    def forward(self, batch, previous, shared, state):
        """`previous` may be None when batch.previous_rows is 0: every row then comes from the state."""
        ops, D = self.ops, self.d_model
        if not batch.n_rows:
            return ops.empty(0, D)
        fused = ops.empty(batch.n_rows, 2 * D)
        ops.gather_rows(previous if previous is not None else state, state, batch.source_index, out=fused[:, :D])
        if hasattr(self.embed_norm, "as_rms"):
            # a norm that offers its (gain, eps) is fused into the gather
            gain, eps = self.embed_norm.as_rms()
            ops.embedding_rmsnorm(shared["embedding"], batch.tokens, gain, eps, out=fused[:, D:])
        else:
            fused[:, D:].copy_(self.embed_norm(ops.embedding(shared["embedding"], batch.tokens)))
        return ops.linear(fused, self.w_proj)

    def after_step(self, batch, previous, state):
        """Once every stage has read its state: the previous stage's newest row of each request waits for the next step."""
        if batch.keep_count:
            self.ops.copy_rows(previous, batch.keep_source, state, batch.keep_slot)
