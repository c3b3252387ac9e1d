from . import arithmatic, batching, bucket, bucket_scope, dev_context, psh_main, subbuck, swin_attn

__all__ = ["arithmatic", "batching", "bucket", "bucket_scope", "dev_context", "psh_main", "subbuck", "swin_attn"]
