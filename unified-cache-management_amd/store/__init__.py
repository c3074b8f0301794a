"""Store-facing side of the block moves: a KV store with the reference's
``UcmKVStoreBase`` surface whose load/dump are single batched HIP launches."""
