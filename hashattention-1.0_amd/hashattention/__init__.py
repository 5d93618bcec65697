"""MI355X-native HashAttention sparse decode: `hashattention.hashattention_llama` / `hashattention_mistral`
expose the reference's module API (`load_usa`, `convert_usa`, `reset_usa`, ...); `_ops` binds the HIP library."""
