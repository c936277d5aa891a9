"""Key/value cache of the decode path, on the HIP entry points.

Mirror of `KVCache` (wrappers/python/nntile/layer/cache_utils.py:117-225) and
of the way `LlamaAttention.forward_dynamic` uses it
(wrappers/python/nntile/model/llama_attention.py:518-531, 643-731): tensors
preallocated with `max_cache_size` rows on the sequence axis, `append` writes
the new rows behind the filled ones, `len()` is the number of filled rows.

What differs, on purpose: the reference copies the filled part of both caches
into fresh dense tensors before every attention call (`k_partial`,
`v_partial`) and materialises a bool mask slice for the new queries; here
`attend` hands the caches to the decode kernel with their capacity and the
visibility rule `key <= query + (len - q_seq)`, so a decode step reads the
filled rows once and writes only the new ones; `append_attend` does the
append and the attention of a decode step in one launch.

Tensors are C-ordered torch device tensors: K, V `[entries, seq, head]`
(entries = n_batch * n_head_kv, NNTile's `[head, seq, n_batch, n_head_kv]`),
Q, A `[entries * kv_group, q_seq, head]`.
"""
import torch

from . import hip_sdpa


class KVCache:
    def __init__(self, max_cache_size, seq_size_dim=1):
        if seq_size_dim != 1:
            # [head, seq, ...] is the only layout the attention path uses
            raise ValueError("the sequence axis of an attention tile is axis 1")
        self.max_cache_size = int(max_cache_size)
        self.seq_size_dim = seq_size_dim
        self.k = None
        self.v = None
        self.k_cache_size = 0
        self.v_cache_size = 0
        self._workspace = None

    def __len__(self):
        return self.k_cache_size

    def _init_from_tensor(self, t):
        entries, _, head = t.shape
        return torch.zeros((entries, self.max_cache_size, head), dtype=t.dtype, device=t.device)

    def append(self, k_partial, v_partial, stream=None):
        """Write the new rows behind the filled ones.  More rows than the cache
        has left raise (the reference raises in
        LlamaAttention._append_to_kv_cache); nothing is written then."""
        if k_partial.shape[1] != v_partial.shape[1]:
            raise ValueError("k and v must bring the same number of tokens")
        if self.k is None:
            self.k = self._init_from_tensor(k_partial)
            self.v = self._init_from_tensor(v_partial)
        rows = k_partial.shape[1]
        if rows + self.k_cache_size > self.max_cache_size:
            raise hip_sdpa.SdpaError(
                hip_sdpa.EINVAL,
                "kv_cache_append: overload internal state: try add %d to %d, max: %d"
                % (rows, self.k_cache_size, self.max_cache_size))
        hip_sdpa.kv_cache_append(k_partial, v_partial, self.k, self.v, self.k_cache_size,
                                 stream=stream)
        self.k_cache_size += rows
        self.v_cache_size += rows

    def append_attend(self, k_partial, v_partial, Q, lse, A, n_batch, kv_group, causal=True,
                      mask=None, stream=None):
        """`append` followed by `attend`, same results bit for bit; on the
        decode kernels' shapes the two are ONE launch (the
        attention reads the new rows from k_partial / v_partial while other
        workgroups of the launch write them into the caches)."""
        rows, q_seq = k_partial.shape[1], Q.shape[1]
        one_launch = (self.k is not None and v_partial.shape[1] == rows
                      and kv_group * q_seq <= 64 and Q.shape[2] in (64, 128)
                      and rows + self.k_cache_size <= self.max_cache_size
                      and k_partial.is_contiguous() and v_partial.is_contiguous())
        if not one_launch:
            self.append(k_partial, v_partial, stream=stream)
            self.attend(Q, lse, A, n_batch, kv_group, causal=causal, mask=mask, stream=stream)
            return
        k_seq = self.k_cache_size + rows
        mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
        sliced = None
        if mask is not None:
            # (the slice that goes with the cache as it will be after the append)
            sliced, mode = self._mask_slice_for(mask, q_seq, k_seq), hip_sdpa.MASK_BOOL
        if stream is not None:
            for t in (sliced, k_partial, v_partial):
                if t is not None:
                    t.record_stream(stream)
        self._mask_in_use = sliced
        workspace = self._decode_workspace(k_seq, Q, n_batch, kv_group, stream)
        hip_sdpa.sdpa_fwd_decode_append_cache(
            k_partial, v_partial, self.k, self.v, k_seq, Q, sliced, lse, A, mode, n_batch, kv_group,
            workspace, causal_offset=k_seq - q_seq, flags=hip_sdpa.OVERWRITE, stream=stream)
        # (only now: a refused call leaves the cache as it was)
        self.k_cache_size += rows
        self.v_cache_size += rows

    def _decode_workspace(self, k_seq, Q, n_batch, kv_group, stream):
        need = hip_sdpa.decode_cache_workspace_bytes(k_seq, Q, n_batch, kv_group)
        if self._workspace is None or self._workspace.numel() < need:
            # (a launch of an earlier call may still read the old workspace:
            # it is kept until the one after next replaces it)
            self._retired_workspace = self._workspace
            self._workspace = torch.empty(need, dtype=torch.uint8, device=Q.device)
        if stream is not None:
            self._workspace.record_stream(stream)
        return self._workspace

    @property
    def k_partial(self):
        """The filled rows, as a view (the reference returns a copy)."""
        return self.k[:, :self.k_cache_size]

    @property
    def v_partial(self):
        return self.v[:, :self.v_cache_size]

    def clear(self):
        self.k = None
        self.v = None
        self.k_cache_size = 0
        self.v_cache_size = 0
        self._workspace = None

    def mask_slice(self, mask, q_seq):
        """The mask rows that go with the last q_seq tokens of the cache
        (Sdpa._prepare_mask_for_kv_cache, wrappers/python/nntile/layer/sdpa.py:
        489-531).  mask: bool device tensor [queries, keys] in C order (the
        reference's [keys, queries]), True = visible.  A mask that already is
        [q_seq, len] is used as it is; otherwise everything is visible except
        where the mask, read at query position len - q_seq + j, says
        otherwise."""
        return self._mask_slice_for(mask, q_seq, len(self))

    @staticmethod
    def _mask_slice_for(mask, q_seq, k_seq):
        if tuple(mask.shape) == (q_seq, k_seq):
            return mask.contiguous()
        out = torch.ones((q_seq, k_seq), dtype=torch.bool, device=mask.device)
        first = k_seq - q_seq
        rows = max(0, min(q_seq, mask.shape[0] - first))
        cols = min(k_seq, mask.shape[1])
        if rows > 0 and cols > 0 and first >= 0:
            out[:rows, :cols] = mask[first:first + rows, :cols]
        return out

    def attend(self, Q, lse, A, n_batch, kv_group, causal=True, mask=None, stream=None):
        """A = attention of Q over the filled rows; the q_seq queries are the
        last q_seq tokens of the cache (append first).  lse and A are
        overwritten.  mask: None (the causal rule when `causal`, else nothing
        hidden) or a bool mask as for `mask_slice`, whose slice is then passed
        as values.  Few rows (kv_group * q_seq <= 64, head 64 or 128) take the
        split-key decode kernel of the tile type, everything else - longer
        chunks, head 32 - the tile kernel; both read the caches in place."""
        k_seq = len(self)
        q_seq = Q.shape[1]
        mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
        sliced = None
        if mask is not None:
            sliced, mode = self.mask_slice(mask, q_seq), hip_sdpa.MASK_BOOL

        def keep(t):
            # The kernels are enqueued through ctypes; torch's allocator does
            # not know they read t.  On a stream other than the current one the
            # allocator is told; in every case the tensor stays referenced
            # here until the next call.
            if stream is not None and t is not None:
                t.record_stream(stream)
            return t

        self._mask_in_use = keep(sliced)
        decode = kv_group * q_seq <= 64 and Q.shape[2] in (64, 128)
        if not decode:
            hip_sdpa.sdpa_fwd_tile_cache(
                self.k, self.v, k_seq, Q, sliced, lse, A, mode, n_batch, kv_group,
                causal_offset=k_seq - q_seq, flags=hip_sdpa.OVERWRITE, stream=stream)
            return
        workspace = self._decode_workspace(k_seq, Q, n_batch, kv_group, stream)
        hip_sdpa.sdpa_fwd_decode_cache(
            self.k, self.v, k_seq, Q, sliced, lse, A, mode, n_batch, kv_group, workspace,
            causal_offset=k_seq - q_seq, flags=hip_sdpa.OVERWRITE, stream=stream)
