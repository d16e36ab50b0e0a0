"""Synthetic inputs generated on the device (seeded SplitMix64 streams)."""
import ctypes

import torch

from . import _lib
from .host import _chk, _ptr, _stream


def words(seed, first, n, device=0):
    out = torch.empty(n, dtype=torch.int64, device=f"cuda:{device}")
    _chk(_lib.load().bam_gen_words(seed, first, n, _ptr(out), _stream()), "bam_gen_words")
    return out


def mod(seed, first, n, modulus, scale=1, device=0):
    out = torch.empty(n, dtype=torch.int64, device=f"cuda:{device}")
    _chk(_lib.load().bam_gen_mod(seed, first, n, modulus, scale, _ptr(out), _stream()), "bam_gen_mod")
    return out


def gather_indices(seed, n, n_elems, first=0, device=0):
    """idx_k = splitmix64(seed ^ 0x5eed, k) mod n_elems"""
    return mod(seed ^ 0x5EED, first, n, n_elems, 1, device)


def block_lbas(seed, n, ns_bytes, req_bytes, lba_bytes, first=0, device=0):
    return mod(seed, first, n, ns_bytes // req_bytes, req_bytes // lba_bytes, device)


def rmat_pairs(seed, scale, first, n, device=0):
    u = torch.empty(n, dtype=torch.int64, device=f"cuda:{device}")
    v = torch.empty(n, dtype=torch.int64, device=f"cuda:{device}")
    _chk(_lib.load().bam_gen_rmat(seed, scale, first, n, _ptr(u), _ptr(v), _stream()), "bam_gen_rmat")
    return u, v


def uniform_pairs(seed, n_vertices, first, n, device=0):
    u = torch.empty(n, dtype=torch.int64, device=f"cuda:{device}")
    v = torch.empty(n, dtype=torch.int64, device=f"cuda:{device}")
    _chk(_lib.load().bam_gen_uniform(seed, n_vertices, first, n, _ptr(u), _ptr(v), _stream()), "bam_gen_uniform")
    return u, v


def build_csr(n_vertices, u, v, chunk=None):
    """Drop self loops, symmetrize, sort, deduplicate; returns (offsets[V+1], neighbours[E]) as int64 device tensors."""
    keep = u != v
    u, v = u[keep], v[keep]
    shift = max(int(n_vertices - 1).bit_length(), 1)
    keys = torch.cat([(u << shift) | v, (v << shift) | u])
    del u, v, keep
    keys = torch.unique(keys)          # sorted + deduplicated
    src = keys >> shift
    dst = keys & ((1 << shift) - 1)
    del keys
    counts = torch.bincount(src, minlength=n_vertices)
    offsets = torch.zeros(n_vertices + 1, dtype=torch.int64, device=dst.device)
    offsets[1:] = torch.cumsum(counts, 0)
    return offsets, dst.contiguous()


def rmat_csr(seed, scale, edge_factor=16, device=0):
    u, v = rmat_pairs(seed, scale, 0, edge_factor << scale, device)
    return build_csr(1 << scale, u, v)


def uniform_csr(seed, n_vertices, n_pairs, device=0):
    u, v = uniform_pairs(seed, n_vertices, 0, n_pairs, device)
    return build_csr(n_vertices, u, v)
