"""A small MI355X-native inference engine for the dense Qwen3 decoder: from a request's tokens to its next token."""

__version__ = "0.1.0"
