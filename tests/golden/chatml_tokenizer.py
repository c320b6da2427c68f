"""A small byte-level ChatML tokenizer for the data-format tests and their fixtures.

Built like the tokenizer of the reference's tests/training/test_maskgit.py:26-43: a byte-level BPE
without merges (one token per byte) plus the special tokens [MASK], <|im_start|>, <|im_end|>, [PAD],
<|image_16383|> and <|image_0..31|>. It offers the four things the MaskGIT transform asks of a
tokenizer (get_vocab, call, decode, pad_token_id) and renders the ChatML template
``<|im_start|>{role}\\n{content}<|im_end|>`` with the assistant mask over an assistant message's
content and closing delimiter.
"""

from __future__ import annotations

from tokenizers import Tokenizer, decoders, pre_tokenizers
from tokenizers.models import BPE

SPECIAL_TOKENS = ["[MASK]", "<|im_start|>", "<|im_end|>", "[PAD]", "<|image_16383|>",
                  *[f"<|image_{i}|>" for i in range(32)]]


class ByteChatTokenizer:
    def __init__(self) -> None:
        alphabet = sorted(pre_tokenizers.ByteLevel.alphabet())
        backend = Tokenizer(BPE({token: index for index, token in enumerate(alphabet)}, []))
        backend.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)
        backend.decoder = decoders.ByteLevel()
        backend.add_special_tokens(SPECIAL_TOKENS)
        self._backend = backend
        self.pad_token_id = backend.token_to_id("[PAD]")

    def __len__(self) -> int:
        return self._backend.get_vocab_size(with_added_tokens=True)

    def get_vocab(self) -> dict[str, int]:
        return self._backend.get_vocab(with_added_tokens=True)

    def __call__(self, text: str) -> dict[str, list[int]]:
        ids = self._backend.encode(text, add_special_tokens=False).ids
        return {"input_ids": list(ids), "attention_mask": [1] * len(ids)}

    def decode(self, ids) -> str:
        return self._backend.decode(list(ids), skip_special_tokens=False)

    def chat(self, messages) -> dict[str, list[int]]:
        """input_ids / attention_mask / assistant_masks of a rendered conversation."""

        ids, assistant = [], []
        for message in messages:
            head = self(f"<|im_start|>{message['role']}\n")["input_ids"]
            body = self(message["content"] + "<|im_end|>")["input_ids"]
            ids += head + body
            assistant += [0] * len(head) + [int(message["role"] == "assistant")] * len(body)
        return {"input_ids": ids, "attention_mask": [1] * len(ids), "assistant_masks": assistant}


def image_grid(width: int = 3, height: int = 2, first: int = 0) -> str:
    return "\n".join("".join(f"<|image_{first + y * width + x}|>" for x in range(width)) for y in range(height))


def record(tokenizer: ByteChatTokenizer, response: str | None = None, prompt: str = "Width: 999 tokens\nHeight: 999 tokens",
           role: str = "assistant") -> dict[str, list[int]]:
    return tokenizer.chat([{"role": "user", "content": prompt},
                           {"role": role, "content": image_grid() if response is None else response}])
