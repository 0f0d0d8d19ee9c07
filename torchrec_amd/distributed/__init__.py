"""Per-shard lookup modules of the sharded inference stack.

Only what runs on one GPU is here: the grouped-table config types, the
fused-parameter keys, and the two modules that wrap one table-batched lookup
operator per shard.  Placement of shards on several GPUs and the exchange of
ids and embeddings between them are not part of this package.
"""
