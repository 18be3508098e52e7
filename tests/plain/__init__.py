"""Plain, slow implementation of the Qwen3 dense decoder in numpy: whole sequences, no cache,
one function per part. It shares no code with the product path and is what the engine is
compared with."""
