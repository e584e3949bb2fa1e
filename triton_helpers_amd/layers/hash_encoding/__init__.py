from .kernel import hash_encoding, hash_encoding_table_grad
from .module import HashEncoding

__all__ = ["hash_encoding", "hash_encoding_table_grad", "HashEncoding"]
