"""KV cache for tree-structured decoding on MI355X.

Replaces umbrella/attn/cache.py (KV_Cache :5-96, StaticKV_Cache :98-192) with one
layout chosen for the HIP attention kernel's MFMA operand loads: inside each
(layer, kv head) slab the elements are stored in FRAGMENT order (round 4;
umbrella_amd/csrc/common.h `kc_off` / `vt_off` are the device-side statement):

    K    slab of Lmax * D elements: a 32-key tile = 2 * (D / 32) fragments of 1 KiB, fragment (s, ds) lane (j, g) holds
         key 32 * tile + 8 * (j / 4) + 4 * s + j % 4, features 32 * ds + 8 * g .. + 7   (A operand of S^T = K Q^T)
    V^T  slab of D * (Lmax + VT_PAD) elements (the first Lmax * D are used): a 32-key tile = D / 16 fragments, fragment dt
         lane (j, g) holds feature 16 * dt + j, keys 32 * tile + 8 * g .. + 7              (A operand of O^T = V^T P^T)

so every load instruction of the attention kernels reads one contiguous KiB (the row-major [Lmax][D] / [D][Lmax] forms gave
16 rows x 64 B per instruction: profiles/r04_attn_frag_probe.txt).  `k_rows` / `v_rows` / `set_rows` and the two
`*_to_frag` / `*_from_frag` pairs convert to and from the semantic [.., Lmax, D] / [.., D, Lmax] views (tests, tools, the
reference-style `gather_kv_incremental`); the hot path never does.

Slots are addressed explicitly (StaticKV semantics); appending is "slot ==
kv_offset".  ``gather_kv_incremental`` keeps the reference signature; the engines
use the device-side ``compact`` (accepted path read from device memory, no tail
memset -- stale slots are never visible because every read is masked by
prefix_len / the tree mask).
"""
from __future__ import annotations

import torch

from .. import _lib

VT_PAD = 32          # == UMB_VT_PAD (include/umbrella_hip.h): slab stride of the V^T cache is D * (Lmax + VT_PAD)


def k_offsets(pos: torch.Tensor, D: int) -> torch.Tensor:
    """element offsets inside a K slab of (key pos[i], feature d) -> LongTensor [len(pos), D]   (common.h kc_off)"""
    p = pos.to(torch.long)[:, None]
    d = torch.arange(D, device=pos.device, dtype=torch.long)[None, :]
    kk = p & 31
    s, j = (kk >> 2) & 1, ((kk >> 3) << 2) | (kk & 3)
    return ((((p >> 5) * 2 + s) * (D >> 5) + (d >> 5)) * 64 + ((d >> 3) & 3) * 16 + j) * 8 + (d & 7)


def vt_offsets(pos: torch.Tensor, D: int) -> torch.Tensor:
    """element offsets inside a V^T slab of (feature d, key pos[i]) -> LongTensor [D, len(pos)]   (common.h vt_off)"""
    p = pos.to(torch.long)[None, :]
    d = torch.arange(D, device=pos.device, dtype=torch.long)[:, None]
    return (((p >> 5) * (D >> 4) + (d >> 4)) * 64 + ((p >> 3) & 3) * 16 + (d & 15)) * 8 + (p & 7)


def k_to_frag(k: torch.Tensor) -> torch.Tensor:
    """semantic K [..., Lmax, D] -> the same shape in fragment order (what the kernels read)"""
    Lmax, D = k.shape[-2:]
    assert Lmax % 32 == 0 and D % 32 == 0
    off = k_offsets(torch.arange(Lmax, device=k.device), D).reshape(-1)
    out = torch.empty_like(k).reshape(*k.shape[:-2], Lmax * D)
    out[..., off] = k.reshape(*k.shape[:-2], Lmax * D)
    return out.reshape(k.shape)


def k_from_frag(ks: torch.Tensor) -> torch.Tensor:
    Lmax, D = ks.shape[-2:]
    off = k_offsets(torch.arange(Lmax, device=ks.device), D).reshape(-1)
    return ks.reshape(*ks.shape[:-2], Lmax * D)[..., off].reshape(ks.shape)


def vt_to_frag(vt: torch.Tensor) -> torch.Tensor:
    """semantic V^T [..., D, Lmax + VT_PAD] -> the same shape, keys 0 .. Lmax-1 in fragment order, the pad tail zero"""
    D, LV = vt.shape[-2:]
    Lmax = LV - VT_PAD
    assert Lmax % 32 == 0 and D % 16 == 0
    off = vt_offsets(torch.arange(Lmax, device=vt.device), D).reshape(-1)
    out = torch.zeros_like(vt).reshape(*vt.shape[:-2], D * LV)
    out[..., off] = vt[..., :Lmax].reshape(*vt.shape[:-2], D * Lmax)
    return out.reshape(vt.shape)


def vt_from_frag(vs: torch.Tensor) -> torch.Tensor:
    D, LV = vs.shape[-2:]
    Lmax = LV - VT_PAD
    off = vt_offsets(torch.arange(Lmax, device=vs.device), D).reshape(-1)
    out = torch.zeros_like(vs)
    out[..., :Lmax] = vs.reshape(*vs.shape[:-2], D * LV)[..., off].reshape(*vs.shape[:-2], D, Lmax)
    return out


class TreeKVCache:
    def __init__(self, num_layers, num_kv_heads, head_dim, max_length, device, dtype):
        assert max_length % 32 == 0, "the fragment-ordered cache is tiled by 32 keys"
        self.num_layers, self.num_key_value_heads, self.head_dim = num_layers, num_kv_heads, head_dim
        self.max_length, self.device, self.dtype = max_length, device, dtype
        # storage (fragment order inside each [layer, head] slab; the shapes only carry the slab strides)
        self.k = torch.zeros(num_layers, num_kv_heads, max_length, head_dim, device=device, dtype=dtype)
        self.vt = torch.zeros(num_layers, num_kv_heads, head_dim, max_length + VT_PAD, device=device, dtype=dtype)
        self.kv_offset = 0

    # ---- semantic access (tests, tools, the reference-style gather): never on the hot path
    def _flat(self):
        L, H = self.num_layers, self.num_key_value_heads
        return self.k.view(L, H, -1), self.vt.view(L, H, -1)

    def k_rows(self, pos) -> torch.Tensor:
        """K of the keys `pos` -> [L, Hkv, len(pos), D]"""
        pos = torch.as_tensor(pos, device=self.device, dtype=torch.long)
        return self._flat()[0][:, :, k_offsets(pos, self.head_dim)]

    def v_rows(self, pos) -> torch.Tensor:
        """V of the keys `pos` -> [L, Hkv, len(pos), D]"""
        pos = torch.as_tensor(pos, device=self.device, dtype=torch.long)
        return self._flat()[1][:, :, vt_offsets(pos, self.head_dim).t()]

    def set_rows(self, pos, k: torch.Tensor, v: torch.Tensor):
        """write K / V [L, Hkv, len(pos), D] at the keys `pos`"""
        pos = torch.as_tensor(pos, device=self.device, dtype=torch.long)
        kf, vf = self._flat()
        kf[:, :, k_offsets(pos, self.head_dim)] = k.to(self.dtype)
        vf[:, :, vt_offsets(pos, self.head_dim).t()] = v.to(self.dtype)

    # reference API (cache.py:41-49): indices are absolute slots, moved to [offset, offset+len)
    def gather_kv_incremental(self, indices, offset: int):
        idx = torch.as_tensor(indices, device=self.device, dtype=torch.long)
        a = idx.numel()
        if a:
            k, v = self.k_rows(idx).clone(), self.v_rows(idx).clone()
            self.set_rows(torch.arange(offset, offset + a, device=self.device), k, v)
        self.kv_offset = offset + a

    def compact(self, result: torch.Tensor, path: torch.Tensor, max_path: int):
        """Device-side compaction driven by umb_accept_scan's outputs (graph-capturable)."""
        _lib.call("umb_kv_compact", self.k, self.vt, result, path, self.num_layers, self.num_key_value_heads,
                  self.head_dim, self.max_length, max_path, _lib.dtype_code(self.dtype))

    def clear(self):
        self.k.zero_()
        self.vt.zero_()
        self.kv_offset = 0

    def set_kv_len(self, kv_len: int):
        self.kv_offset = kv_len


class PagedSeqCache:
    """Paged key/value store, pooled blocks and recurrent-state slots for MANY sequences (the sequence-mixer models of
    libumbrella_seq.so; device-side statement: csrc/seq_common.h ``pkv_tok`` / ``pkv_blk``).

    * a sequence holds a SLOT (a row of the page table and of every recurrent-state array) from ``open`` to ``close``;
    * its tokens live in PAGES of ``page`` positions handed out on demand by ``extend`` and returned by ``close``; the same
      page numbers index every windowed-attention layer's K / V ``[pages, G, page, D]`` (storage dtype) and its pooled K / V
      ``[pages, G, ceil(page / pool), D]`` (fp32; a block lives in the page of its last position);
    * latent-attention layers keep ONE row per token, ``[pages, page, kv_rank + rot_dim]`` (storage dtype): the normed
      key/value latent and the rotated key part that all heads share;
    * gated-linear-attention layers keep one fp32 state ``[slots, H, D, Dv]`` each;
    * a convolution in front of a sublayer keeps its last ``taps - 1`` inputs, fp32 ``[slots, taps - 1, W]`` per sublayer
      (the input at position p in row p % (taps - 1)); a mixer's own input convolution does the same over its own channels
      (``mixer_convs``: ``(taps, channels)`` each);
    * softmax-attention layers with separate values keep K ``[pages, G, page, D]`` and V ``[pages, G, page, E]`` and no
      pooled entries (a ``kv_layers`` entry ``(G, D, 0, E)``);
    * element-wise recurrences use the same state arrays with ``(1, 1, channels)``;
    * nothing is cleared when a slot or a page is handed out again: a sequence that starts at position 0 ignores what its
      slot holds, and no kernel reads a cache position its own sequence has not written.

    Free pages and slots are LIFO stacks, so whatever was given back last is used first.
    """

    def __init__(self, kv_layers, state_layers, max_tokens: int, max_seqs: int, device, dtype, page: int = 64,
                 latent_layers=(), conv_states: int = 0, conv_taps: int = 0, width: int = 0, mixer_convs=()):
        assert page >= 1 and max_tokens >= 1 and max_seqs >= 1
        self.page, self.max_seqs, self.device, self.dtype = int(page), int(max_seqs), device, dtype
        # every sequence may leave one page partly filled
        self.n_pages = (max_tokens + page - 1) // page + max_seqs
        self.max_pages = self.n_pages
        self.pages_dev = torch.zeros(max_seqs, self.max_pages, dtype=torch.int32, device=device)
        self.kv, self.state = [], []
        for spec in kv_layers:
            G, D, pool = spec[:3]
            E = spec[3] if len(spec) > 3 else D                         # value size (pooled layers: the key size)
            entry = dict(k=torch.zeros(self.n_pages, G, page, D, dtype=dtype, device=device),
                         v=torch.zeros(self.n_pages, G, page, E, dtype=dtype, device=device), kp=None, vp=None, G=G, D=D, E=E,
                         pool=pool)
            if pool > 0:
                npb = (page + pool - 1) // pool
                entry["kp"] = torch.zeros(self.n_pages, G, npb, D, dtype=torch.float32, device=device)
                entry["vp"] = torch.zeros(self.n_pages, G, npb, D, dtype=torch.float32, device=device)
            self.kv.append(entry)
        for (H, D, Dv) in state_layers:
            self.state.append(torch.zeros(max_seqs, H, D, Dv, dtype=torch.float32, device=device))
        self.latent = [torch.zeros(self.n_pages, page, Dk, dtype=dtype, device=device) for Dk in latent_layers]
        self.conv = [torch.zeros(max_seqs, max(conv_taps - 1, 1), width, dtype=torch.float32, device=device)
                     for _ in range(conv_states)] if conv_taps > 0 else []
        self.mixer_conv = [torch.zeros(max_seqs, max(taps - 1, 1), ch, dtype=torch.float32, device=device)
                           for (taps, ch) in mixer_convs]
        self.clear()

    def clear(self):
        self.free_pages = list(range(self.n_pages - 1, -1, -1))
        self.free_slots = list(range(self.max_seqs - 1, -1, -1))
        self.seqs = {}                                   # id -> {"slot", "len", "pages"}

    # ---- bookkeeping (host)
    def open(self, seq_id) -> int:
        if seq_id in self.seqs:
            raise KeyError(f"sequence {seq_id!r} is already open")
        if not self.free_slots:
            raise RuntimeError(f"no free sequence slot ({self.max_seqs} in use)")
        slot = self.free_slots.pop()
        self.seqs[seq_id] = dict(slot=slot, len=0, pages=[])
        return slot

    def close(self, seq_id):
        s = self.seqs.pop(seq_id)
        self.free_pages.extend(reversed(s["pages"]))
        self.free_slots.append(s["slot"])

    def length(self, seq_id) -> int:
        return self.seqs[seq_id]["len"]

    def slot(self, seq_id) -> int:
        return self.seqs[seq_id]["slot"]

    def tokens_held(self) -> int:
        return sum(s["len"] for s in self.seqs.values())

    def can_extend(self, seq_id, n: int) -> bool:
        s = self.seqs[seq_id]
        need = (s["len"] + n + self.page - 1) // self.page - len(s["pages"])
        return need <= len(self.free_pages)

    def extend(self, seq_id, n: int) -> int:
        """Reserve room for the next n positions of a sequence; returns its first new position.  The page-table row on
        the device is updated (stream-ordered) before the caller's next launch."""
        s = self.seqs[seq_id]
        pos0 = s["len"]
        need = (pos0 + n + self.page - 1) // self.page - len(s["pages"])
        if need > len(self.free_pages):
            raise RuntimeError(f"paged cache exhausted: {need} pages wanted, {len(self.free_pages)} free "
                               f"({self.n_pages} pages of {self.page} tokens)")
        if need > 0:
            have = len(s["pages"])
            new = [self.free_pages.pop() for _ in range(need)]
            s["pages"].extend(new)
            self.pages_dev[s["slot"], have:have + need] = torch.tensor(new, dtype=torch.int32).to(self.device, non_blocking=False)
        s["len"] = pos0 + n
        return pos0

    # ---- semantic access (tests, tools): never on the hot path
    def token_rows(self, layer: int, seq_id, positions):
        """cached (K, V) of a sequence's positions -> two tensors [len(positions), G, D]"""
        s, c = self.seqs[seq_id], self.kv[layer]
        pos = torch.as_tensor(positions, dtype=torch.long)
        pg = torch.tensor(s["pages"], dtype=torch.long)[pos // self.page].to(self.device)
        off = (pos % self.page).to(self.device)
        return c["k"][pg, :, off], c["v"][pg, :, off]

    def pooled_rows(self, layer: int, seq_id, blocks):
        """pooled (K, V) of a sequence's blocks -> two fp32 tensors [len(blocks), G, D]"""
        s, c = self.seqs[seq_id], self.kv[layer]
        e = torch.as_tensor(blocks, dtype=torch.long) * c["pool"] + c["pool"] - 1
        pg = torch.tensor(s["pages"], dtype=torch.long)[e // self.page].to(self.device)
        idx = ((e % self.page) // c["pool"]).to(self.device)
        return c["kp"][pg, :, idx], c["vp"][pg, :, idx]

    def latent_rows(self, layer: int, seq_id, positions):
        """cached latent rows of a sequence's positions -> [len(positions), kv_rank + rot_dim]"""
        s = self.seqs[seq_id]
        pos = torch.as_tensor(positions, dtype=torch.long)
        pg = torch.tensor(s["pages"], dtype=torch.long)[pos // self.page].to(self.device)
        return self.latent[layer][pg, (pos % self.page).to(self.device)]

    def latent_struct(self, layer: int) -> "_lib.UmbPagedKV":
        kv = _lib.UmbPagedKV()
        kv.k, kv.v, kv.kp, kv.vp = self.latent[layer].data_ptr(), None, None, None
        kv.pages, kv.max_pages, kv.page, kv.n_pages = self.pages_dev.data_ptr(), self.max_pages, self.page, self.n_pages
        return kv

    def struct(self, layer: int) -> "_lib.UmbPagedKV":
        c = self.kv[layer]
        kv = _lib.UmbPagedKV()
        kv.k, kv.v = c["k"].data_ptr(), c["v"].data_ptr()
        kv.kp, kv.vp = (c["kp"].data_ptr(), c["vp"].data_ptr()) if c["kp"] is not None else (None, None)
        kv.pages, kv.max_pages, kv.page, kv.n_pages = self.pages_dev.data_ptr(), self.max_pages, self.page, self.n_pages
        return kv
