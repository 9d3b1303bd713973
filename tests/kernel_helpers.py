"""Helpers of the kernel tests: paged caches built from dense keys and values, and the plain
references the kernels are compared with."""

import torch

import plain_llama


def make_paged(ks, vs, block_size, dtype, seed=0, spare_pages=3, poison=True):
    """ks[b], vs[b]: [S_b, n_kv, D].  Returns k_pool [pages, n_kv, bs, D], v_pool [pages, n_kv, D, bs]
    (values transposed inside a page), block_tables int32 [B, M]; pages in shuffled order, the
    unused slots filled with NaN."""
    n_kv, d = ks[0].shape[1:]
    need = [-(-k.shape[0] // block_size) for k in ks]
    pages = sum(need) + spare_pages
    g = torch.Generator().manual_seed(seed)
    order = torch.randperm(pages, generator=g).tolist()
    fill = float("nan") if poison else 0.0
    k_pool = torch.full((pages, n_kv, block_size, d), fill, dtype=dtype)
    v_pool = torch.full((pages, n_kv, d, block_size), fill, dtype=dtype)
    tables = torch.zeros((len(ks), max(need)), dtype=torch.int32)
    for b, (k, v) in enumerate(zip(ks, vs)):
        for i in range(need[b]):
            page = order.pop()
            tables[b, i] = page
            chunk = slice(i * block_size, min((i + 1) * block_size, k.shape[0]))
            n = chunk.stop - chunk.start
            k_pool[page, :, :n] = k[chunk].transpose(0, 1).to(dtype)
            v_pool[page, :, :, :n] = v[chunk].permute(1, 2, 0).to(dtype)
    return k_pool, v_pool, tables


def attention_reference(q_full, k, v, rows, window=None):
    """q_full [S, nh, D] (queries of every position), k/v [S, nkv, D]; returns [len(rows), nh*D] float32
    of the plain causal attention at the given positions."""
    out = plain_llama.causal_attention(q_full.float().transpose(0, 1), k.float().transpose(0, 1),
                                       v.float().transpose(0, 1), window)  # [nh, S, D]
    return out.transpose(0, 1)[rows].reshape(len(rows), -1)


def bf16_round(x):
    return x.to(torch.bfloat16).float()
