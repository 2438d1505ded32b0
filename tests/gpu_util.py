"""Helpers of the GPU tests: scatter whole sequences into a paged cache with arbitrary page ids."""
import os
import random

import torch

DEV = os.environ.get("ULLM_TEST_DEVICE", "cuda:0")


def tol(dtype, ref):
    """Allowed max abs difference: relative to the largest reference value."""
    scale = float(ref.abs().max())
    return (3e-2 if dtype == torch.bfloat16 else 2e-5) * scale + 1e-6


def paged_cache(seqs_k, seqs_v, page_size, dtype, device, spare_pages=3, seed=0, fill=None):
    """seqs_k/v: list of [S_b, nkv, hd] float tensors.  Returns k_pool [pages, nkv, P, hd], v_pool
    [pages, nkv, hd, P] (values are transposed inside a page) and
    block tables (list of page-id lists) with page ids shuffled; unused rows hold ``fill`` (NaN by
    default so that any read of them shows)."""
    nkv, hd = seqs_k[0].shape[1:]
    n_pages = sum(-(-k.shape[0] // page_size) for k in seqs_k) + spare_pages
    ids = list(range(n_pages))
    random.Random(seed).shuffle(ids)
    fillv = float("nan") if fill is None else fill
    k_pool = torch.full((n_pages, nkv, page_size, hd), fillv, dtype=torch.float32)
    v_pool = torch.full((n_pages, nkv, hd, page_size), fillv, dtype=torch.float32)
    tables = []
    for k, v in zip(seqs_k, seqs_v):
        table = []
        for i in range(-(-k.shape[0] // page_size)):
            page = ids.pop()
            table.append(page)
            rows = k[i * page_size:(i + 1) * page_size]
            k_pool[page, :, :rows.shape[0]] = rows.transpose(0, 1)
            v_pool[page, :, :, :rows.shape[0]] = v[i * page_size:(i + 1) * page_size].permute(1, 2, 0)
        tables.append(table)
    return k_pool.to(device, dtype), v_pool.to(device, dtype), tables


def table_tensor(tables, device, stride=None):
    stride = stride or max(len(t) for t in tables)
    bt = torch.full((len(tables), stride), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        bt[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
    return bt.to(device)
