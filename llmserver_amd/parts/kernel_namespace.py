"""What the parts, the step function and the engine ask of the object that carries the kernels (``ctx.ops``).

The package ships one such object, ``llmserver_amd.kernels.HipOps`` (hand-written HIP for gfx950); the tests pass
plain torch twins in its place.  Both derive from :class:`KernelNamespace`, which names every call: the ones every
namespace must answer raise ``NotImplementedError`` here, and the ones that only a namespace with fused or tuned
kernels answers have neutral answers here ("not offered"), so that no caller has to ask whether a method exists.
"""
from __future__ import annotations

import contextlib
from typing import Optional


class KernelNamespace:
    name = ""                       # "hip": the step function may record single-token steps into graphs
    fuse_stream_updates = False     # the few-row products fold the residual sum and the norm around them in
    fuses_bias = False              # linear() and linear_few_rows() take a bias themselves (one rounding)
    attention_tuning = None         # an AttentionTuning for this GPU, or None: the attention part's neutral defaults

    # -- what every namespace must do (shapes and meanings: see HipOps, whose docstrings are the contract) -----------
    def preload(self, head_dims, dtype) -> None:
        """Load (compile, if need be) what models of these head sizes and this type will call."""

    def linear(self, x, weight, out=None, out_float32=False, bias=None, bias_rounded=None):
        raise NotImplementedError

    def embedding(self, table, token_ids, out):
        raise NotImplementedError

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None):
        raise NotImplementedError

    def swiglu(self, gate_up, out, activation="silu"):
        """``out = act(gate) * up`` with ``gate_up [T, 2I]``, gate first; a namespace refuses an ``activation`` it has not built."""
        raise NotImplementedError

    def add_bias_(self, y, bias):
        raise NotImplementedError

    def rotary_table(self, positions, inv_freq):
        raise NotImplementedError

    def qk_norm_rope_kv_write(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin,
                              page_size, n_q, n_kv, head_dim, write_cache=True):
        raise NotImplementedError

    def paged_attention(self, qkv, out, keys, values, table, row_start, row_len, row_ctx, plan, scale, window, page_size,
                        n_q, n_kv, head_dim, ctx, decode_fusion=None, sinks=None, softcap=None):
        """``sinks [n_q]`` (float32) or None: one more term ``exp(sinks[head])`` in every softmax's denominator, with no
        key and no value.  ``softcap`` (a number or None): scaled scores become ``softcap * tanh(score / softcap)`` before
        the mask.  ``qkv`` may hold the queries only (``[T, n_q * head_dim]``) where nothing is fused."""
        raise NotImplementedError

    def qkv_prepare(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin, page_size,
                    n_q, n_kv, dim, value_dim, out_q, write_cache=True, pairing="neighbours"):
        """``qkv [T, n_q * dim + n_kv * dim + n_kv * value_dim]``.  Per head, queries and keys are RMS-normed over ``dim``
        (``q_weight`` / ``k_weight [dim]`` float32, or both None: no norm), then the first ``2 * pairs`` dimensions turn
        in neighbouring pairs (2i, 2i+1) or, with ``pairing="halves"``, in pairs (i, i + pairs), by ``cos_sin [T, 2 * pairs]``
        (cosines, then sines; None: no rotation).  With
        ``D`` the pages' head size: ``out_q [T, n_q * D]`` gets the query rows, zeros behind ``dim``; with ``write_cache``,
        ``keys [pages, n_kv, page_size, D]`` get the key rows and ``values [pages, n_kv, D, page_size]`` the value rows
        (zeros behind ``dim`` / ``value_dim``) at every token's place."""
        raise NotImplementedError

    # Recurrent mixers.
    def token_shift(self, h, mu, state, offset, state_slots, token_row, positions, row_start, out, keep=False):
        """``out[m, t] = h[t] + (before[t] - h[t]) * mu[m]``, ``mu [M, W]`` float32, ``out [M, T, W]`` of ``h``'s type.
        ``before[t]``: the row of the token before ``t`` in its request: a row of this step, or, for a row's first
        token, ``state[slot, offset : offset + W]`` (float32; zeros at position 0 whatever the state holds).  ``keep``
        (steps of one token per row only): the state also becomes this step's row, as :meth:`token_shift_keep` would do."""
        raise NotImplementedError

    def token_shift_keep(self, h, state, offset, state_slots, row_start, row_len):
        """``state[slot, offset : offset + W] =`` every row's last row of ``h`` (rows without tokens keep theirs)."""
        raise NotImplementedError

    def batched_linear(self, x, weights):
        """``x [B, T, in]``, ``weights [B, out, in]`` -> ``[B, T, out]`` of ``x``'s type, 32-bit sums."""
        raise NotImplementedError

    def tanh_(self, x):
        raise NotImplementedError

    def linear_recurrence(self, q, k, v, decay, decay_bias, decay_mode, tau, bonus, q_scale, state, offset, state_slots,
                          row_start, row_len, row_ctx, out, heads, dim, value_dim):
        """Per row (request) and head, over the row's tokens in order: ``d_t = decay(decay[t] + decay_bias)`` per key
        channel (``"sigmoid_root"``: ``sigmoid(z)^(1/tau)``; ``"double_exp"``: ``exp(-exp(z))``), all float32.  ``bonus``
        None: ``S = diag(d_t) S + k_t v_t^T``, ``out_t = S^T (q_t * q_scale)``.  ``bonus [heads, dim]``:
        ``out_t = (S + diag(bonus) k_t v_t^T)^T (q_t * q_scale)``, then ``S = diag(d_t) S + k_t v_t^T``.
        ``q, k [T, heads * dim]``, ``v [T, heads * value_dim]`` (views with unit stride along a row), ``decay [T, heads *
        dim]`` float32, ``out [T, heads * value_dim]`` float32.  ``S [heads, dim, value_dim]`` float32 lies in
        ``state[slot, offset:]``; a row whose first token stands at position 0 starts from zeros whatever the slot holds;
        the state after the row's last token is stored back."""
        raise NotImplementedError

    def heads_norm_gate(self, x, weight, weight_per_channel, eps, gate, out, heads, value_dim, gate_activation="silu", below=None, floor=0.0):
        """``out[t, h, :] = x'[t, h, :] / rms(x'[t, h, :]) * w * act(gate[t, h, :])``; ``x`` float32, ``w = weight [value_dim]``
        shared by the heads or, with ``weight_per_channel``, ``weight [heads * value_dim]``; ``gate`` a view like ``out``;
        ``act``: ``"silu"`` or ``"sigmoid"``.  ``x' = x``, or, with ``below [T, heads, 2]`` (float32):
        ``x / (max(|below[..., 0]|, below[..., 1]) + floor)``, a matrix memory's read-out under its normaliser."""
        raise NotImplementedError

    def matrix_memory_chunks(self, n_tokens, rows):
        """0: a step of this shape runs its matrix memories token by token.  Otherwise the memories run in chunks (matrix
        products over a chunk's tokens) and want scratch memory for this many chunks (``matrix_memory``'s ``run``, ``sums``)."""
        return 0

    def matrix_memory(self, q, k, v, gates, cap, q_scale, state, state_slots, row_start, row_len, row_ctx, out, below, coefficients,
                      heads, dim, value_dim, run=None, sums=None):
        """A matrix memory with exponential gates, per row (request) and head over the row's tokens in order, all float32.
        ``gates [T, 2 * heads]``: the input gates' logits, then the forget gates'.  ``i = cap * tanh(z_i / cap)``,
        ``f = logsigmoid(cap * tanh(z_f / cap))``, ``m_t = max(f + m_(t-1), i)``, ``keep = exp(f + m_(t-1) - m_t)``,
        ``take = exp(i - m_t)``; ``S_t = keep S_(t-1) + take k_t v_t^T``, ``n_t = keep n_(t-1) + take k_t``.
        ``out [T, heads * value_dim] = S_t^T (q_t * q_scale)`` (the numerators only), ``below [T, heads, 2] =
        (n_t . (q_t * q_scale), exp(-m_t))``, ``coefficients [T, heads, 2]`` scratch (keep, take).  ``q, k [T, heads * dim]``,
        ``v [T, heads * value_dim]`` (views with unit stride along a row).  ``state[slot]``: ``S [heads, dim, value_dim]``,
        then ``n [heads, dim]``, then ``m [heads]``; a row whose first token stands at position 0 starts from zeros whatever
        the slot holds; the state after the row's last token is stored back.  ``run`` (float64 ``[T, heads]``) and ``sums``
        (float32 ``[chunks, heads, dim, value_dim + 1]``): scratch memory of the chunked form, given when
        ``matrix_memory_chunks`` said so."""
        raise NotImplementedError

    # Several residual streams in 32-bit.
    def streams_read(self, streams, read, weight, eps, out, rows=None):
        """``out = rmsnorm(sum_s read[s] * streams[s, rows]) * weight``; ``streams [S, T, W]`` float32, ``rows`` int32 or None
        (all); ``out`` of any type."""
        raise NotImplementedError

    def streams_update(self, streams, y, mix, write, next_read=None, next_weight=None, next_eps=0.0, normed=None):
        """Where they lie, every new stream from the streams as they stood before: ``streams[t] <- sum_s mix[s, t] * streams[s] + write[t] * y``
        (``y [T, W]`` of any type).  With ``next_read``: ``normed = rmsnorm(sum_t next_read[t] * streams[t]) * next_weight``
        of the new streams (eps ``next_eps``, any type)."""
        raise NotImplementedError

    def activation_(self, x, activation):
        """``x = act(x)`` where it lies, in 32-bit, rounded once: ``"relu2"`` (``max(x, 0)^2``), ``"gelu_tanh"``, ``"silu"``."""
        raise NotImplementedError

    def linear_activated(self, x, weight, activation):
        """``act(x @ weight^T)`` in ``x``'s type, ``act`` as in :meth:`activation_`, computed on the product's 32-bit sums
        where the kernel that forms them can (one rounding), on the rounded product otherwise."""
        raise NotImplementedError

    def scaled_sum(self, x, x_scale, y, y_scale, out):
        raise NotImplementedError

    # A residual stream kept in 32-bit beside activations of the compute type.
    def embedding_norm(self, table, token_ids, weight, eps, out):
        """``out [T, W]`` float32 ``= rmsnorm(table[token_ids]) * weight``."""
        raise NotImplementedError

    def embedding_wide(self, table, token_ids, out, scale=1.0):
        """``out [T, W]`` float32 ``= table[token_ids] * scale``; an ``out [S, T, W]`` gets the rows ``S`` times."""
        raise NotImplementedError

    def norm_add_norm(self, x, y, weight, eps, out, next_weight=None, next_eps=0.0, normed=None, y2=None, scales=None):
        """``out = x + rmsnorm(y') * weight`` in float32, with ``y' = y`` or, with ``y2`` and ``scales = (a, b)``,
        ``a * y + b * y2``; with ``next_weight``: ``normed = rmsnorm(out) * next_weight`` (eps ``next_eps``, any type)."""
        raise NotImplementedError

    def norm_rows(self, x, rows, weight, eps, out):
        """``out = rmsnorm(x[rows]) * weight`` for a float32 ``x``; ``rows`` int32 or None (all); ``out`` of any type."""
        raise NotImplementedError

    def short_conv(self, x, weight, state, state_slots, token_row, positions, row_start, out, keep=False):
        """``out = x + conv(x)``: a causal convolution over each request's tokens on every channel, ``weight [W, taps]``,
        tap ``j`` on the token ``taps - 1 - j`` places back; tokens before the step's come from ``state [slots, taps - 1,
        W]`` (a request's last inputs, oldest first), tokens before the sequence are zeros.  ``x`` float32.  ``keep``
        (steps of one token per row only): the state also moves on by the step's token, as :meth:`short_conv_keep` would do."""
        raise NotImplementedError

    def short_conv_keep(self, x, state, state_slots, row_start, row_len, row_ctx):
        """Move every row's last ``taps - 1`` inputs (the step's, and the state's where the step brings fewer) into ``state``."""
        raise NotImplementedError

    def scaled_norm_add(self, x, y, weight, scale, eps, out, rounded=None, history=None, before=0, mix=None):
        """``s = x + rmsnorm(y) * weight * scale`` (``scale`` None: 1), all float32.  Without ``history``: ``out = s``.
        With ``history [states, T, W]``: ``history[before] = s`` and ``out = sum_{j <= before} mix[j] * history[j]``.
        ``rounded`` (any type) also gets ``out``."""
        raise NotImplementedError

    # Attention over a shared low-rank latent.
    def latent_prepare(self, proj, q_latent, norm_weight, eps, cos_sin, keys, values, table, token_row, positions, page_size,
                       out_q, n_heads, dim, rot_dim, rank, write_cache=True, up_keys=None):
        """``proj [T, n_heads * (dim + rot_dim) + rank + rot_dim + ...]``: per head ``dim`` plain and ``rot_dim`` rotated
        query dimensions, then the token's ``rank`` latent dimensions and its ``rot_dim`` shared rotated key dimensions.
        Writes a cache row ``[rmsnorm(latent) * norm_weight, rotate(key part), zeros]`` of every token as its key and,
        transposed, as its value, and ``out_q [T, n_heads * D]`` with per head ``[q_latent[h, t], rotate(q's rotated part),
        zeros]``.  ``cos_sin [T, 2 * pairs]``: neighbouring dimensions (2i, 2i+1) of the first ``2 * pairs`` rotated ones turn.
        ``q_latent`` None and ``up_keys [heads, dim, rank]`` given: ``q_latent[h, t] = q_plain[t, h] @ up_keys[h]`` is made here."""
        raise NotImplementedError

    def gate_heads(self, y, proj, gate_column, out, mixed=None, up_values=None, per_channel=False):
        """``out[t, h * v + j] = y[h, t, j] * sigmoid(proj[t, gate_column + h])`` (``gate_column`` < 0: no gate; ``per_channel``:
        a gate for every channel, ``proj[t, gate_column + h * v + j]``).  ``y`` None and
        ``mixed [T, heads * row]``, ``up_values [heads, rank, v]`` given: ``y[h, t] = mixed[t, h, :rank] @ up_values[h]`` is made here."""
        raise NotImplementedError

    # A block whose sublayers' results join the stream together under sigmoid gates.
    def gated_pair_update(self, x, gates, y1, scale1, y2, scale2, next_weight=None, next_eps=0.0, normed=None):
        """``x += scale1 * sigmoid(gates[:, :W]) * y1 + scale2 * sigmoid(gates[:, W:]) * y2`` in float32, where it lies
        (``y2``, ``scale2`` None: one sublayer, ``gates [T, W]``); ``y`` of any type; with ``next_weight``:
        ``normed = rmsnorm(x) * next_weight`` (eps ``next_eps``, any type)."""
        raise NotImplementedError

    # Differential attention: the two maps' results behind the attention kernels.
    def differential_heads(self, attended, lam, keep, eps, out, kv_heads, group, value_dim, row):
        """``attended [T, kv_heads * 2 * group * row]``: for key/value head ``g`` the results of map 1 of its ``group`` query
        heads, then of map 2, each in a row of ``row`` numbers of which ``value_dim`` count.  ``out[t, (g * group + r) *
        value_dim + j] = d / sqrt(mean_j(d^2) + eps) * keep`` with ``d = a1 - lam * a2``."""
        raise NotImplementedError

    # The gated delta rule.
    def delta_prepare(self, proj, taps, state, offset, state_slots, token_row, positions, row_start, out, kv_heads, heads, dim,
                      value_dim, q_scale, unit_eps, strength, decay, decay_scale, decay_bias, per_channel, out_strength, out_decay,
                      keep=False):
        """The first ``C = 2 * kv_heads * dim + heads * value_dim`` columns of ``proj`` (queries, keys, values) pass a causal
        convolution over each request's tokens per channel (``taps [C, K]``, tap ``j`` on the token ``K - 1 - j`` places
        back, zeros before the sequence, earlier steps' inputs from ``state[slot, offset:]`` as ``[K - 1, C]``, oldest first)
        and silu; every query and key head is then divided by ``sqrt(sum of its squares + unit_eps)``, queries also times
        ``q_scale``.  ``out [T, C]`` float32.  Beside them ``out_strength [T, heads] = sigmoid(strength)`` and
        ``out_decay = exp(-exp(decay_scale[h]) * softplus(decay + decay_bias))`` with ``decay [T, heads]`` and ``decay_bias
        [heads]``, or, ``per_channel``, ``decay [T, heads * dim]`` float32 and ``decay_bias [heads * dim]``.  ``keep`` (steps of
        one token per row only): the state also moves on by the step's token, as :meth:`delta_conv_keep` would do."""
        raise NotImplementedError

    def delta_conv_keep(self, proj, channels, taps, state, offset, state_slots, row_start, row_len, row_ctx):
        """Move every row's last ``taps - 1`` inputs of the convolutions (the step's, and the state's where the step brings
        fewer) into ``state[slot, offset:]``."""
        raise NotImplementedError

    def delta_rule(self, prepared, strength, decay, per_channel, state, offset, state_slots, row_start, row_len, row_ctx, out,
                   heads, kv_heads, dim, value_dim):
        """Per head ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q`` over each row's tokens, with
        ``prepared [T, C]``, ``strength [T, heads]`` (beta) and ``decay`` (g: ``[T, heads]``, or, ``per_channel``, ``[T, heads *
        dim]``, a decay for every row of ``S``) from :meth:`delta_prepare`; head ``h`` reads query/key head ``h // (heads /
        kv_heads)``.  ``S`` lives in ``state[slot, offset:]`` in float32 as blocks of 16 value columns, ``[heads, ceil(value_dim /
        16), dim, 16]``; zeros before a sequence's first token.  ``out [T, heads * value_dim]`` float32."""
        raise NotImplementedError

    # Routed experts.
    def route_experts(self, x, router, top, chosen, weights, scoring="softmax", groups=None, bias=None):
        """Float32 logits ``x router^T``; ``chosen [T, top]`` the largest (first of equals), ``weights`` their softmax.
        ``scoring="sigmoid"``: scores ``sigmoid(logits)``, the largest scores chosen, the scores themselves the weights;
        ``groups=(count, keep)``: only experts of the ``keep`` best of ``count`` equal groups of neighbours can be chosen,
        a group's score the sum of its two largest scores (the first of equal groups).  ``bias [experts]`` joins the logits."""
        raise NotImplementedError

    def experts_gate_up(self, x, gate_up, chosen, hidden, activation="silu", limit=0.0):
        """``hidden[t * top + s] = silu(G x_t) * (U x_t)`` with ``[G; U] = gate_up[chosen[t, s]]`` (``[E, 2F, W]``);
        ``activation="clamped"``: ``g = min(G x, limit)``, ``u = clamp(U x, -limit, limit)``, ``g * sigmoid(1.702 g) * (u + 1)``."""
        raise NotImplementedError

    def experts_down(self, hidden, down, chosen, weights, out):
        """``out[t] = sum_s weights[t, s] * down[chosen[t, s]] hidden[t * top + s]``; ``down [E, W, F]``, ``out`` float32."""
        raise NotImplementedError

    def sample(self, logits, temperature, uniform, out):
        raise NotImplementedError

    # -- what a namespace may offer; the answers here mean "not offered" --------------------------------------------
    def latent_products_inside(self, n_tokens: int) -> bool:
        """Whether, for a step of this many tokens, :meth:`latent_prepare` and :meth:`gate_heads` should make the per-head
        products themselves (``up_keys=`` / ``up_values=``) instead of getting them from batched products made before."""
        return False

    def experts_sorted(self, x, gate_up, down, chosen, weights, out, activation="silu", limit=0.0) -> bool:
        """Both products of the routed experts and the weighted sum for all of the step's tokens at once, the (token,
        expert) pairs sorted by expert so that an expert's matrices are read once per tile of pairs: ``out`` as
        :meth:`experts_down` leaves it.  False: not done (not offered, or it would not pay for these sizes)."""
        return False

    def check_cache_geometry(self, cache_specs, page_size: int, num_pages=None) -> None:
        """Raise ``ValueError`` for a cache that the kernels cannot read (asked before anything is allocated):
        ``page_size`` keys a page, ``num_pages`` pages (one number, or one per group of caches; None: not said)."""

    def row_scale_fits(self, x, weight, row_scale) -> bool:
        """Whether the few-row product of these sizes can apply a norm as a scale of its rows."""
        return False

    def linear_few_rows(self, x, weight, out=None, out_float32=False, rows_per_workgroup=0, row_scale=None, bias=None):
        """The weight-streaming product (taking a pending norm as ``row_scale``), or None: no case for it."""
        return None

    def linear_into_stream(self, x, weight, resid, norm_weight, rows_per_workgroup=0, row_scale=None):
        """The product as an update of the residual stream with the following norm prepared, or None."""
        return None

    def linear_partial_sums(self, x, weight, few_rows_too=False):
        """The product as float32 partial sums ``[parts, T, out]`` for :meth:`add_rmsnorm` to add up, or None."""
        return None

    def partial_sums_are_faster(self, x, weight) -> bool:
        return False

    def library_is_faster(self, kind, x, weight, scaled=False, out_float32=False) -> bool:
        return False

    def linear_gated(self, x, gate_up_weight, pairs_per_workgroup=0, row_scale=None, activation="silu"):
        """Gate and up products with the activation in one launch, or None (also for an ``activation`` it has not built)."""
        return None

    def attention_tuning_for(self, dtype, head_dim=None):
        """``attention_tuning`` as it holds for tensors of ``dtype`` and heads of ``head_dim`` (kernels of different types
        may step through their keys differently, and costs grow with the head); here: the same for all."""
        return self.attention_tuning

    def attention_workgroup_tiles(self, dtype, head_dim, page_size=None) -> int:
        """Most tiles a workgroup of a prompt-portion attention kernel takes together; 0: there is no such kernel."""
        return 0

    def attention_tile_halves(self, dtype, head_dim) -> int:
        return 1

    def attention_tile_key_ranges(self, dtype, head_dim) -> int:
        """Most ranges the keys of a workgroup's tiles may be cut into for workgroups of their own (1: not offered)."""
        return 1

    def attention_tile_min_workgroups(self, dtype) -> int:
        return 0

    def decode_fusion_fits(self, dtype, head_dim) -> bool:
        """Whether ``paged_attention`` takes q/k norm, rotation and the cache write on itself in single-token steps."""
        return False

    def measuring(self):
        """A context in which unknown shapes may be timed and entered into a table of choices; here: nothing happens."""
        return contextlib.nullcontext(None)


def tuning_of(ops: KernelNamespace, default, dtype=None, head_dim=None):
    """The namespace's attention tuning for steps of this type and head size, or ``default`` where it has none."""
    tuning: Optional[object] = ops.attention_tuning_for(dtype, head_dim) if dtype is not None else ops.attention_tuning
    return tuning if tuning is not None else default
