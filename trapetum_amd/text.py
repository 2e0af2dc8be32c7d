"""Text in and out for the command line, when a model folder holds a tokenizer.json.

The library itself works on token ids.  The reference's server encodes a prompt with its folder's tokenizer.json
and no special tokens of its own (chat templates are applied before: runtime/src/bin/serve.rs:145, :312) and
decodes the whole continuation at once, since one character may be split over tokens (serve.rs:341-345); the
command line here does the same through the `tokenizers` package, which is a tokenizer library and holds no model
code.  Without that file, or without the package, text prompts are refused with an error that says so.
"""
import os


class TextError(RuntimeError):
    pass


class FolderTokenizer:
    def __init__(self, folder):
        path = os.path.join(folder, "tokenizer.json")
        if not os.path.exists(path):
            raise TextError(f"{folder} has no tokenizer.json: give the prompt as token ids (--prompt-ids, or a file of int32 ids)")
        try:
            from tokenizers import Tokenizer
        except ImportError as e:
            raise TextError(f"a text prompt needs the `tokenizers` package: {e}") from None
        self._tok = Tokenizer.from_file(path)

    def encode(self, text):
        """Token ids of `text`, no special tokens added (serve.rs:312 encodes with add_special_tokens = false)."""
        ids = self._tok.encode(text, add_special_tokens=False).ids
        if not ids:
            raise TextError("the prompt encodes to no token")
        return list(ids)

    def decode(self, ids):
        return self._tok.decode(list(ids), skip_special_tokens=True)
