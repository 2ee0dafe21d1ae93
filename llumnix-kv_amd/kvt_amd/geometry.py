"""The cache geometry the Python connector hands to the transfer client, as
closed forms over tensor shapes (what ParseBlock's WorkerInfo is filled from):

* token_bytes per cache tensor     blade_kvt/hybrid_connector/kvtbackend.py:1012-1046
* block_bytes                      blade_kvt/hybrid_connector/kvtbackend.py:1048-1059
* layer_num_blocks                 blade_kvt/kv_transfer_impl.py:105-139

Shapes are plain tuples and sizes plain integers: nothing here needs torch."""


def token_bytes(cache_shapes, elem_sizes):
    """cache_shapes: the distinct per-layer KV tensor shapes (one entry in the normal case,
    two 3-D shapes for the sparse-MLA layout with an indexer cache); elem_sizes: bytes per
    element of each. -> list of token sizes, one per shape."""
    shapes = [tuple(s) for s in cache_shapes]
    if len(shapes) != len(elem_sizes) or not shapes:
        raise ValueError("one element size per cache shape is required")
    if len(shapes) == 1:
        shape = shapes[0]
        if len(shape) == 5:
            # FlashAttention [2, nblk, bs, h, d] or FlashInfer [nblk, 2, bs, h, d] (for the HND
            # stride order the logical shape is the same): K and V rows of all heads
            return [2 * shape[3] * shape[4] * elem_sizes[0]]
        if len(shape) != 3:
            raise ValueError("expected a 5-D attention cache or a 3-D MLA cache, got %r" % (shape,))
        return [shape[2] * elem_sizes[0]]      # MLA: [nblk, bs, kv_lora_rank + rope_dim]
    out = []
    for shape, elem in zip(shapes, elem_sizes):
        if len(shape) != 3:
            raise ValueError("several shapes per layer are only supported for 3-D (sparse MLA) "
                             "caches, got %r" % (shape,))
        out.append(shape[2] * elem)
    return out


def block_bytes(token_sizes, block_size, attn_pack_size=1, hybrid=False):
    """A registered hybrid attention tensor is a physical page bundling attn_pack_size
    consecutive attention layers."""
    pack = attn_pack_size if hybrid else 1
    return [t * block_size * pack for t in token_sizes]


def layer_num_blocks(layer_nbytes, block_nbytes):
    """layer_nbytes: byte size of every registered layer tensor (all must agree)."""
    if block_nbytes <= 0:
        raise ValueError("block_bytes must be positive, got %d" % block_nbytes)
    sizes = list(layer_nbytes)
    for i, n in enumerate(sizes):
        if n != sizes[0]:
            raise ValueError("all registered KV layers must have identical layout; layer %d has "
                             "%d bytes, expected %d" % (i, n, sizes[0]))
        if n % block_nbytes != 0:
            raise ValueError("KV layer size is not divisible by block_bytes; layer %d: %d %% %d"
                             % (i, n, block_nbytes))
    return sizes[0] // block_nbytes
