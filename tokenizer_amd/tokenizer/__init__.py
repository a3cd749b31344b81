from .qwen_bpe import Tokenizer, TokenizerError, UnknownToken, bytes_to_unicode_reverse

__all__ = ["Tokenizer", "TokenizerError", "UnknownToken", "bytes_to_unicode_reverse"]
