"""A second construction of the block description of a CSR pattern, with torch operations
(sorts, uniques, scatters) instead of the device kernels: what tests compare
scorch_hip_csr_block_count / scorch_hip_csr_block_fill and the lists built from them against.
Test infrastructure only; runs on whatever device its inputs live on."""
import torch


def describe(pos: torch.Tensor, crd: torch.Tensor, M: int, n_cols: int):
    """dict of block_row_ptr, block_col_idx, block_words, block_off, block_cols, block_nnz for a
    pattern whose rows hold strictly increasing columns."""
    block = 64
    nbr, nbc = M // block, n_cols // block
    dev = pos.device
    nnz = int(crd.numel())
    pos64, crd64 = pos.to(torch.int64), crd.to(torch.int64)
    rows = torch.repeat_interleave(torch.arange(M, device=dev, dtype=torch.int64), pos64[1:] - pos64[:-1],
                                   output_size=nnz)
    blocks, block_of = torch.unique(rows // block * nbc + crd64 // block, return_inverse=True)
    n_active = int(blocks.numel())
    key = block_of * block + rows % block
    words = torch.zeros(n_active * block, dtype=torch.int64, device=dev)
    words.index_add_(0, key, torch.ones_like(crd64) << (crd64 % block))     # distinct bits: the sum is the union
    first = torch.full((n_active * block,), nnz, dtype=torch.int64, device=dev)
    first.scatter_reduce_(0, key, torch.arange(nnz, device=dev, dtype=torch.int64), "amin")
    first[first == nnz] = 0
    used = words.view(n_active, block)
    while used.shape[1] > 1:
        used = used[:, 0::2] | used[:, 1::2]
    stored = torch.zeros(n_active, dtype=torch.int64, device=dev).index_add_(0, block_of, torch.ones_like(crd64))
    block_row_ptr = torch.zeros(nbr + 1, dtype=torch.int64, device=dev)
    block_row_ptr[1:] = torch.cumsum(torch.bincount(blocks // nbc, minlength=nbr), 0)
    return {"block_row_ptr": block_row_ptr.to(torch.int32), "block_col_idx": (blocks % nbc).to(torch.int32),
            "block_words": words, "block_off": first.to(torch.int32), "block_cols": used.reshape(-1).contiguous(),
            "block_nnz": stored.to(torch.int32)}


def stretches(lens, longest, split_slots):
    """Work items by plain loops: (items, split_rows, n_slots) as lists of tuples."""
    items, split_rows, at, slot = [], [], 0, 0
    for row, n in enumerate(lens):
        n = int(n)
        if n <= longest:
            items.append((n, row, at, at + n, -1 if split_slots else 0))
        else:
            parts = -(-n // longest)
            if split_slots:
                split_rows.append((row, slot, parts, 0))
            for part in range(parts):
                lo, hi = at + n * part // parts, at + n * (part + 1) // parts
                items.append((hi - lo, row, lo, hi, slot if split_slots else 0))
                slot += 1
        at += n
    items.sort(key=lambda it: -it[0])
    return [it[1:] for it in items], split_rows, slot if split_slots else 0
