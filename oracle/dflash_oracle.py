"""CPU oracle for the DFlash speculative-verify hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module: it is the checker the HIP kernels are compared against, used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.  It is a plain numpy restatement of the reference's *ops*
implementations (the code SwiftLM runs when the default device is the CPU or
``DFLASH_FORCE_OPS`` is set) and of the host-side accept / commit / rollback
indexing.  Each function cites the reference lines it follows.

The arithmetic underneath the reference's ops path lives in MLX (SharpAI/mlx via
SharpAI/mlx-swift, a path dependency of Package.swift:16 whose version is not
pinned and whose sources are absent from the reference tree).  MLX's own
reduction order and rounding points are therefore not reproduced bit for bit;
the functions below compute in a caller-chosen dtype (float32 mirrors the ops
path after type promotion, float64 gives a ground truth for tolerance checks).

Pinning status (what fixes each function other than its own formula):

* ``tape_replay_ops``            closed form for scalar gates, prefix
                                 composition, identities, fp64 brute force.
* ``gated_delta_ops_with_tape``  textbook delta rule in matrix form
                                 ``S <- g S (I - b k k^T) + b v k^T``, the
                                 in-tree second restatement
                                 (Sources/SwiftLM/KimiLinearDFlash.swift:383-405),
                                 forward/replay consistency, special cases.
* masked variants                equal the unmasked function on the sub-sequence
                                 of unmasked steps.
* ``match_acceptance_length``    the reference's own documented example
                                 (DFlashRuntime.swift:130-132) + brute force.
* ``rebuild_conv_state``, ``restore_target_cache_after_acceptance``,
  ``accept_commit``              integer indexing, brute force.
* ``sdpa_block_causal``          library softmax / logsumexp (scipy), row-sum
                                 invariants, reduction to plain causal attention.
* ``sdpa_2pass``                 must agree with ``sdpa_block_causal``.

The reference holds no golden vectors for any of these (its only numeric check
is Metal-vs-ops ``cos > 0.999 and max_abs_diff < 0.01``,
tests/DFlash/DFlashProfiler.swift:215-244), so the bit-level behaviour of MLX on
this path is "parity unpinned"; everything is held to the stated tolerances.
"""

from __future__ import annotations

import numpy as np

# ----------------------------------------------------------------------------
# bf16 / f16 helpers (numpy has no bfloat16)
# ----------------------------------------------------------------------------


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bfloat16 (ties to even); returns float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    nan = np.isnan(x)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32).copy()
    out[nan] = np.nan
    return out.reshape(x.shape)


def round_to_f16(x: np.ndarray) -> np.ndarray:
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def quantize(x: np.ndarray, dtype: str | None) -> np.ndarray:
    """Round to ``dtype`` ('f32' | 'bf16' | 'f16' | None) and return in x's dtype."""
    if dtype in (None, "f32", "f64"):
        return x
    if dtype == "bf16":
        return round_to_bf16(x.astype(np.float32)).astype(x.dtype)
    if dtype == "f16":
        return round_to_f16(x.astype(np.float32)).astype(x.dtype)
    raise ValueError(dtype)


# ----------------------------------------------------------------------------
# a1  tape replay
# ----------------------------------------------------------------------------


def _repeat_heads(x: np.ndarray, rf: int) -> np.ndarray:
    # MLX.repeated(k, count: rf, axis: 2): consecutive repeat, value head hv
    # reads key head hv // rf (DFlashKernels.swift:384 and :47).
    return np.repeat(x, rf, axis=2) if rf > 1 else x


def tape_replay_ops(tape, k, g, state, mask=None, *, dtype=np.float32, requant=None):
    """Replay an innovation tape through the recurrent state.

    Follows ``tapeReplayOps`` (Sources/DFlash/DFlashKernels.swift:371-407):
    for each step ``state = state * decay + delta * k``, with ``decay`` the
    multiplicative gate (scalar per head ``[B,T,Hv]`` or per channel
    ``[B,T,Hv,Dk]``), and a masked step leaving the state untouched
    (``MLX.where(stepMask, state, prev)``, :399-403).

    ``requant`` ('bf16' | 'f16') re-rounds the state after every step, which
    is what the Metal kernel does for a low-precision state
    (DFlashKernels.swift:70); None follows the ops path.

    Shapes: tape [B,T,Hv,Dv], k [B,T,Hk,Dk], state [B,Hv,Dv,Dk], mask [B,T].
    """
    tape = np.asarray(tape, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    g = np.asarray(g, dtype=dtype)
    state = np.asarray(state, dtype=dtype).copy()
    T = tape.shape[1]
    Hk, Hv = k.shape[2], tape.shape[2]
    k = _repeat_heads(k, Hv // Hk)
    for t in range(T):
        prev = state
        if g.ndim == 4:
            decay = g[:, t, :, None, :]
        else:
            decay = g[:, t, :, None, None]
        delta = tape[:, t, :, :, None]
        kT = k[:, t, :, None, :]
        state = quantize(state * decay + delta * kT, requant)
        if mask is not None:
            step = (np.asarray(mask)[:, t] > 0.5)[:, None, None, None]
            state = np.where(step, state, prev)
    return state


# ----------------------------------------------------------------------------
# a2  gated delta forward with tape
# ----------------------------------------------------------------------------


def gated_delta_ops_with_tape(q, k, v, g, beta, state, mask=None, *, dtype=np.float32,
                              requant=None):
    """GatedDelta forward that also records the innovation tape.

    Follows ``gatedDeltaOpsWithTape`` (DFlashKernels.swift:409-466): per step
    ``S' = S*decay``; ``kv_mem = sum_dk S'*k``; ``delta = (v - kv_mem)*beta``;
    ``S = S' + k (x) delta``; ``y = sum_dk S*q``.  A masked step keeps S and
    emits y = 0 and delta = 0 (:446-453).

    ``requant`` ('bf16' | 'f16') follows the Metal kernel for a low-precision state
    (:148-199): the state is re-rounded to the storage type after every executed step
    (:183-186), while that step's y is read from the state before the rounding (:171-172).

    Returns (y [B,T,Hv,Dv], state [B,Hv,Dv,Dk], tape [B,T,Hv,Dv] float32).
    """
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    g = np.asarray(g, dtype=dtype)
    beta = np.asarray(beta, dtype=dtype)
    state = np.asarray(state, dtype=dtype).copy()
    B, T, Hk, Dk = q.shape
    Hv = v.shape[2]
    q = _repeat_heads(q, Hv // Hk)
    k = _repeat_heads(k, Hv // Hk)
    ys, tapes = [], []
    for t in range(T):
        if g.ndim == 4:
            decay = g[:, t, :, None, :]
        else:
            decay = g[:, t, :, None, None]
        decayed = state * decay
        kt = k[:, t, :, None, :]
        kv_mem = (decayed * kt).sum(axis=-1)
        delta = (v[:, t] - kv_mem) * beta[:, t, :, None]
        updated = decayed + kt * delta[..., None]
        # The Metal kernel reads y out of the updated state BEFORE it re-rounds that state to the
        # storage type (DFlashKernels.swift:171-172, rounding at :183-186); without requant the two coincide.
        y = (updated * q[:, t, :, None, :]).sum(axis=-1)
        new_state = quantize(updated, requant)
        if mask is not None:
            step = np.asarray(mask)[:, t] > 0.5
            sg = step[:, None, None, None]
            yg = step[:, None, None]
            state = np.where(sg, new_state, state)
            ys.append(np.where(yg, y, 0))
            tapes.append(np.where(yg, delta, 0))
        else:
            state = new_state
            ys.append(y)
            tapes.append(delta)
    y = np.stack(ys, axis=1)
    tape = np.stack(tapes, axis=1)
    if dtype == np.float32:
        tape = tape.astype(np.float32)
    return y, state, tape


# ----------------------------------------------------------------------------
# a5 / a6  acceptance length and commit indexing
# ----------------------------------------------------------------------------


# ---------------------------------------------------------------------------
# GatedDelta pre-ops: short causal conv + SiLU, q/k normalisation, gate formulas
# (the layer code around the recurrence: Sources/SwiftLM/KimiLinearDFlash.swift)
# ---------------------------------------------------------------------------

def short_conv_silu(x, conv_state, weight):
    """``ShortConv1d`` (KimiLinearDFlash.swift:274-293): depthwise causal conv over
    ``concat(state, x)`` along time, then SiLU.  x [B,T,C]; conv_state [B,K-1,C] or
    None (zeros, :288); weight [C,K] (tap j multiplies the row j steps into the
    window).  Returns (out [B,T,C], new_state [B,K-1,C] = the last K-1 rows of the
    concatenation, :292)."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(weight, dtype=np.float64)
    B, T, C = x.shape
    K = w.shape[1]
    prev = np.zeros((B, K - 1, C)) if conv_state is None else np.asarray(conv_state, dtype=np.float64)
    ci = np.concatenate([prev, x], axis=1)                       # [B, T+K-1, C]
    out = np.zeros((B, T, C))
    for j in range(K):
        out += ci[:, j:j + T, :] * w[None, None, :, j]
    out = out / (1.0 + np.exp(-out))                             # silu (:291)
    return out, ci[:, T:, :]


def rms_norm_scaled(x, scale, eps=1e-6):
    """``scale * rmsNorm(x, weight: none, eps)`` over the last axis (KimiLinearDFlash.swift:362-363)."""
    x = np.asarray(x, dtype=np.float64)
    return scale * x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def gdn_gates(a_logits, b_logits, a_log, dt_bias):
    """``g = exp(-exp(A_log) * softplus(a + dt_bias))``, ``beta = sigmoid(b)``
    (KimiLinearDFlash.swift:390-391).  a_logits [B,T,H] with dt_bias [H], or
    [B,T,H,Dk] with dt_bias [H,Dk]; a_log [H]."""
    a = np.asarray(a_logits, dtype=np.float64)
    al = np.asarray(a_log, dtype=np.float64)
    db = np.asarray(dt_bias, dtype=np.float64)
    if a.ndim == 4:
        al = al[:, None]
        db = db.reshape(a.shape[2], a.shape[3])
    z = a + db
    softplus = np.logaddexp(0.0, z)
    g = np.exp(-np.exp(al) * softplus)
    beta = 1.0 / (1.0 + np.exp(-np.asarray(b_logits, dtype=np.float64)))
    return g, beta


def gdn_prepare(mixed_qkv, conv_state, conv_weight, a_logits, b_logits, a_log, dt_bias,
                Hk, Hv, Dk, Dv, q_scale, k_scale, eps=1e-6):
    """The layer's steps between its projections and the recurrence
    (KimiLinearDFlash.swift:351-364, :390-391) on the concatenated q|k|v channels:
    conv+SiLU, split, ``q = q_scale * rmsNorm(q)``, ``k = k_scale * rmsNorm(k)`` per head,
    gates.  Returns dict(q, k, v, g, beta, conv_state)."""
    out, new_state = short_conv_silu(mixed_qkv, conv_state, conv_weight)
    B, T, _ = out.shape
    cq = Hk * Dk
    q = rms_norm_scaled(out[..., :cq].reshape(B, T, Hk, Dk), q_scale, eps)
    k = rms_norm_scaled(out[..., cq:2 * cq].reshape(B, T, Hk, Dk), k_scale, eps)
    v = out[..., 2 * cq:].reshape(B, T, Hv, Dv)
    g, beta = gdn_gates(a_logits, b_logits, a_log, dt_bias)
    return dict(q=q, k=k, v=v, g=g, beta=beta, conv_state=new_state)


def gdn_finish(y, gate, norm_weight, eps, gate_kind="sigmoid"):
    """``rmsNorm(y; weight, eps) * act(gate)`` over the last axis (KimiLinearDFlash.swift:377-378,
    RMSNorm :341); act = sigmoid, or silu for the gated RMSNorm variant."""
    y = np.asarray(y, dtype=np.float64)
    z = np.asarray(gate, dtype=np.float64)
    n = y / np.sqrt((y * y).mean(axis=-1, keepdims=True) + eps) * np.asarray(norm_weight, dtype=np.float64)
    sig = 1.0 / (1.0 + np.exp(-z))
    return n * (z * sig if gate_kind == "silu" else sig)


def build_suppress_token_mask(vocab_size: int, suppress_token_ids):
    """Boolean [vocab] mask of the in-range ids, or None when there are none
    (DFlashRuntime.swift:105-115)."""
    ids = sorted({int(i) for i in (suppress_token_ids or []) if 0 <= int(i) < vocab_size})
    if not ids:
        return None
    mask = np.zeros(vocab_size, dtype=bool)
    mask[ids] = True
    return mask


def greedy_tokens_with_mask(logits, suppress_token_mask=None, *, dtype="f32"):
    """``argmax(where(mask, -1e9 as logits.dtype, logits), axis=-1)`` as uint32
    (DFlashRuntime.swift:118-128).  ``dtype`` names the logits' type: the floor is
    -1e9 ROUNDED to it (bf16: -999292928).  The first index wins a tie (numpy's
    argmax rule; the array library's own argMax is not in the reference tree)."""
    x = np.asarray(logits, dtype=np.float32)
    if suppress_token_mask is not None:
        floor = np.float32(-1e9)
        if dtype == "bf16":
            floor = round_to_bf16(np.array([floor], np.float32))[0]
        elif dtype == "f16":
            with np.errstate(over="ignore"):
                floor = np.float32(np.float16(floor))       # -inf: -1e9 overflows float16
        x = np.where(np.asarray(suppress_token_mask, dtype=bool), floor, x)
    return np.argmax(x, axis=-1).astype(np.uint32)


def match_acceptance_length(drafted, posterior) -> int:
    """Number of leading positions where drafted == posterior.

    ``sum(cumprod(drafted == posterior))``; empty input gives 0
    (Sources/DFlash/DFlashRuntime.swift:133-142).
    """
    drafted = np.asarray(drafted).reshape(-1)
    posterior = np.asarray(posterior).reshape(-1)
    if drafted.shape[0] == 0:
        return 0
    matches = (drafted == posterior[: drafted.shape[0]]).astype(np.int32)
    return int(np.cumprod(matches).sum())


def accept_commit(staged_first: int, drafted, posterior, start: int):
    """One verify cycle's integer bookkeeping (DFlashRuntime.swift:484-581).

    ``drafted`` are the block's draft tokens *after* the staged first token
    (length V-1); ``posterior`` the target's greedy tokens for all V verify
    positions.  Returns a dict with the reference's names.
    """
    drafted = np.asarray(drafted).reshape(-1)
    posterior = np.asarray(posterior).reshape(-1)
    verify_ids = np.concatenate([[staged_first], drafted]).astype(np.int64)   # :490-493
    V = verify_ids.shape[0]
    if V > 1:
        acceptance_len = match_acceptance_length(verify_ids[1:], posterior[: V - 1])  # :525-530
    else:
        acceptance_len = 0
    commit_count = 1 + acceptance_len                                          # :544
    committed = verify_ids[:commit_count]                                      # :545
    staged_next = int(posterior[acceptance_len])                               # :547
    new_start = start + commit_count                                           # :571
    return {
        "acceptance_len": acceptance_len,
        "commit_count": commit_count,
        "committed": committed,
        "staged_next": staged_next,
        "start": new_start,
        # arguments handed to engine.rollback (:573-578)
        "rollback_args": {"target_len": new_start, "acceptance_length": acceptance_len,
                          "drafted_tokens": V - 1},
    }


# ----------------------------------------------------------------------------
# a3  rollback cache
# ----------------------------------------------------------------------------


def rebuild_conv_state(snapshot_conv, tape_qkv, accepted_steps: int, keep: int = 3):
    """Conv window after accepting ``accepted_steps`` tokens.

    ``concat([snapshot_conv, tape_qkv], axis=1)[:, s : min(s + keep, len)]``
    with ``s = accepted_steps`` (RecurrentRollbackCache.swift:139-158).  A
    missing snapshot counts as ``keep`` rows of zeros (:147-152).
    """
    tape_qkv = np.asarray(tape_qkv)
    if keep <= 0:
        return None
    if snapshot_conv is None:
        snapshot_conv = np.zeros((tape_qkv.shape[0], keep, tape_qkv.shape[-1]), tape_qkv.dtype)
    conv_input = np.concatenate([np.asarray(snapshot_conv), tape_qkv], axis=1)
    start = accepted_steps
    end = min(start + keep, conv_input.shape[1])
    return conv_input[:, start:end]


class RecurrentRollbackCacheOracle:
    """State machine of ``RecurrentRollbackCache`` (RecurrentRollbackCache.swift:34-182)."""

    def __init__(self, conv_kernel_size: int = 4):
        self.keep = conv_kernel_size - 1
        self.slots = [None, None]          # [conv state, recurrent state]
        self.offset = 0
        self.armed = False
        self._tape = self._k = self._g = self._qkv = None
        self._snapshot = None

    def arm_rollback(self, prefix_len: int = 0):            # :63-71
        self.armed = True
        self._tape = self._k = self._g = self._qkv = None
        self._snapshot = [self.slots[0], self.slots[1]]

    def record_tape(self, tape, k, g, qkv):                 # :75-85
        self._tape, self._k, self._g, self._qkv = tape, k, g, qkv

    def rollback(self, n_accepted: int, *, dtype=np.float32):  # :95-131
        if self._snapshot is None:
            self.clear_transients()
            return
        snap = self._snapshot
        if snap[0] is not None:
            self.slots[0] = snap[0]
        if snap[1] is not None:
            self.slots[1] = snap[1]
        if self._tape is not None and self._k is not None and self._g is not None \
                and self.slots[1] is not None:
            steps = n_accepted + 1                           # :115
            self.slots[1] = tape_replay_ops(self._tape[:, :steps], self._k[:, :steps],
                                            self._g[:, :steps], self.slots[1], dtype=dtype)
            if self._qkv is not None:
                self.slots[0] = rebuild_conv_state(snap[0], self._qkv, steps, self.keep)
        self.clear_transients()

    def clear_transients(self):                              # :163-170
        self.armed = False
        self._tape = self._k = self._g = self._qkv = None
        self._snapshot = None

    def trim(self, n: int) -> int:                           # :175-181
        trimmed = min(self.offset, n)
        self.offset -= trimmed
        return trimmed


def restore_target_cache_after_acceptance(caches, target_len, acceptance_length, drafted_tokens):
    """Per-cache action list of ``restoreTargetCacheAfterAcceptance``.

    (Sources/DFlash/DFlashRuntime.swift:188-223.)  ``caches`` is a list of
    ``(kind, offset)`` with kind in {'rollback', 'mamba', 'kv'}; returns, per
    cache, one of ('clear',), ('rollback', n_accepted), ('set_offset', n),
    ('trim', n), ('none',).
    """
    fully = drafted_tokens > 0 and acceptance_length == drafted_tokens
    out = []
    for kind, offset in caches:
        if kind == "rollback":
            out.append(("clear",) if fully else ("rollback", acceptance_length))
        elif kind == "mamba":
            out.append(("set_offset", target_len))
        elif kind == "kv":
            out.append(("trim", offset - target_len) if offset > target_len else ("none",))
        else:
            raise ValueError(kind)
    return out


# ----------------------------------------------------------------------------
# a8  block-causal GQA SDPA
# ----------------------------------------------------------------------------


def sdpa_block_causal(q, k, v, scale, mask=None, *, dtype=np.float64):
    """``softmax(scale * Q K^T + causal [+ mask]) V`` for a draft block.

    Q [B,Hq,M,D]; K,V [B,Hk,N,D] where N already includes the M block tokens;
    row i sees keys ``0 .. N-M+i`` (DFlashKernels.swift:614).  GQA head mapping
    ``hk = hq // (Hq/Hk)`` (:575).  ``mask`` is an optional additive
    [B,Hq,M,N] (:548-553); -inf entries drop the key, a row left without keys
    yields zeros (:711).  Returns (O [B,Hq,M,D], lse [B,Hq,M]) in ``dtype``;
    ``lse = max + log(sum exp)`` of the scaled, masked scores (natural log).

    This is what ``sdpaFallback`` (:818-828) asks of
    MLXFast.scaledDotProductAttention when handed the same causal mask.
    """
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    rf = Hq // Hk
    out = np.empty((B, Hq, M, v.shape[3]), dtype=dtype)
    lse = np.empty((B, Hq, M), dtype=dtype)
    rows = np.arange(M)[:, None]
    cols = np.arange(N)[None, :]
    visible = cols <= (N - M + rows)
    for b in range(B):
        for h in range(Hq):
            hk = h // rf
            s = (q[b, h] * dtype(scale)) @ k[b, hk].T          # scale folded into Q (:594)
            if mask is not None:
                mk = np.asarray(mask[b, h], dtype=dtype)
                # a key is used only when its mask value is a finite number of the input type (:551);
                # the mask value is added to the score (:553)
                s = np.where(mk > -np.inf, s + mk, -np.inf)
            s = np.where(visible, s, -np.inf)
            m = s.max(axis=-1, keepdims=True)
            m_safe = np.where(np.isfinite(m), m, 0.0)
            p = np.exp(s - m_safe)
            l = p.sum(axis=-1, keepdims=True)
            with np.errstate(divide="ignore", invalid="ignore"):
                out[b, h] = np.where(l > 0, (p @ v[b, hk]) / np.where(l > 0, l, 1.0), 0.0)   # no usable key: zeros (:711)
                lse[b, h] = np.where(l > 0, m_safe + np.log(l), -np.inf)[:, 0]
    return out, lse


def gather_pages(pool, page_table, n_keys: int):
    """Dense [B, Hk, n_keys, D] view of a paged cache: pool [num_pages, Hk, page_size, D],
    page_table [B, pages]; key n of sequence b is row n % page_size of page page_table[b, n // page_size].
    The reference keeps its cache dense (what batchedSDPA2Pass receives, DFlashKernels.swift:737-743);
    this is the layout transform that relates the paged entry to it."""
    pool = np.asarray(pool)
    page_table = np.asarray(page_table)
    ps = pool.shape[2]
    n = np.arange(n_keys)
    pages = page_table[:, n // ps]                      # [B, n_keys]
    return np.transpose(pool[pages, :, (n % ps)[None, :]], (0, 2, 1, 3))


def scatter_pages(dense, page_table, num_pages: int, page_size: int, fill=0.0):
    """Inverse of gather_pages: a pool that holds dense [B, Hk, N, D] under page_table."""
    dense = np.asarray(dense)
    B, Hk, N, D = dense.shape
    pool = np.full((num_pages, Hk, page_size, D), fill, dtype=dense.dtype)
    for b in range(B):
        for n in range(N):
            pool[page_table[b][n // page_size], :, n % page_size] = dense[b, :, n]
    return pool


def sdpa_2pass(q, k, v, scale, blocks=32, *, partial_dtype="bf16"):
    """Restatement of the reference's split-KV two-pass kernels in float32.

    Pass 1 (DFlashKernels.swift:563-649): block ``b`` of ``blocks`` walks keys
    ``b, b+blocks, ...`` with an online softmax and stores an unnormalised
    partial O rounded to the input type (:647) plus fp32 max / sum.
    Pass 2 (:661-720): global max, rescaled sum, weighted partial sum, divide
    unless the sum is 0.  Returns O float32 [B,Hq,M,D] (before the final cast).
    """
    q = np.asarray(q, dtype=np.float32)
    k = np.asarray(k, dtype=np.float32)
    v = np.asarray(v, dtype=np.float32)
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    rf = Hq // Hk
    fmin = np.finfo(np.float32).min
    out = np.zeros((B, Hq, M, D), np.float32)
    for b in range(B):
        for h in range(Hq):
            hk = h // rf
            qs = np.float32(scale) * q[b, h]
            part = np.zeros((M, blocks, D), np.float32)
            sums = np.zeros((M, blocks), np.float32)
            maxs = np.full((M, blocks), fmin, np.float32)
            for blk in range(blocks):
                idx = np.arange(blk, N, blocks)
                if idx.size == 0:
                    continue
                s = qs @ k[b, hk, idx].T                               # [M, n_blk]
                use = idx[None, :] <= (N - M + np.arange(M)[:, None])
                s = np.where(use, s, -np.inf)
                mx = np.maximum(s.max(axis=-1), fmin)
                p = np.where(use, np.exp(s - mx[:, None]), 0).astype(np.float32)
                sums[:, blk] = p.sum(axis=-1)
                maxs[:, blk] = mx
                part[:, blk] = quantize((p @ v[b, hk, idx]).astype(np.float32), partial_dtype)
            gmax = maxs.max(axis=-1)
            w = np.exp(maxs - gmax[:, None]).astype(np.float32)
            tot = (w * sums).sum(axis=-1)
            o = (w[:, :, None] * part).sum(axis=1)
            out[b, h] = np.where(tot[:, None] == 0, o, o / np.where(tot == 0, 1, tot)[:, None])
    return out


# ----------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations
# ----------------------------------------------------------------------------


def _softplus(x):
    return np.log1p(np.exp(-np.abs(x))) + np.maximum(x, 0)


def make_gdn_inputs(seed, B, T, Hk, Hv, Dk, Dv, *, in_dtype="f32", vec_gate=False):
    """q,k L2-normalised N(0,1); v N(0,1); beta sigmoid(N(0,1)); g = exp(-softplus(N(0,1)))
    (the multiplicative decay the kernels take); state N(0, 0.1).  Inputs are rounded to
    ``in_dtype`` and returned as float32; the state stays float32."""
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, T, Hk, Dk)).astype(np.float32)
    k = rng.standard_normal((B, T, Hk, Dk)).astype(np.float32)
    q /= np.linalg.norm(q, axis=-1, keepdims=True)
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    v = rng.standard_normal((B, T, Hv, Dv)).astype(np.float32)
    beta = (1.0 / (1.0 + np.exp(-rng.standard_normal((B, T, Hv))))).astype(np.float32)
    gshape = (B, T, Hv, Dk) if vec_gate else (B, T, Hv)
    g = np.exp(-_softplus(rng.standard_normal(gshape))).astype(np.float32)
    state = (0.1 * rng.standard_normal((B, Hv, Dv, Dk))).astype(np.float32)
    q, k, v, beta, g = (quantize(a, in_dtype) for a in (q, k, v, beta, g))
    return dict(q=q, k=k, v=v, beta=beta, g=g, state=state)


def draw_accepted(rng, T, kind="uniform"):
    """The benchmark's accepted length n in [1, T]: uniform (config 0) or Geometric(0.25) clipped."""
    if kind == "uniform":
        return int(rng.integers(1, T + 1))
    return int(min(rng.geometric(0.25), T))


def make_sdpa_inputs(seed, B, Hq, Hk, M, L, D):
    """bf16-rounded N(0,1) Q [B,Hq,M,D], K,V [B,Hk,L+M,D] as float32."""
    rng = np.random.default_rng(seed)
    q = round_to_bf16(rng.standard_normal((B, Hq, M, D)).astype(np.float32))
    k = round_to_bf16(rng.standard_normal((B, Hk, L + M, D)).astype(np.float32))
    v = round_to_bf16(rng.standard_normal((B, Hk, L + M, D)).astype(np.float32))
    return q, k, v
