"""Symbol table with the reference's special-symbol layout
(metaseq/data/dictionary.py:22-42: <s>=0, <pad>=1, </s>=2, <unk>=3).  The generator asks it
for the pad / unk / eos ids, the vocabulary size, and - for factual-nucleus sampling - the ids
of ".", "?" and "!" (metaseq/sequence_generator.py:116)."""
from typing import Dict, Optional


class Dictionary:
    def __init__(self, vocab_size: int, bos=0, pad=1, eos=2, unk=3,
                 symbols: Optional[Dict[str, int]] = None, tokenizer=None):
        """``symbols`` maps textual symbols to ids (the vocabulary file's content);
        ``tokenizer`` is anything with ``token_to_id(str)`` (a Hugging Face ``tokenizers``
        object).  Without either, no textual symbol can be resolved: ``index`` returns unk and
        ``resolves`` says so."""
        self._n = int(vocab_size)
        self.bos_index, self.pad_index, self.eos_index, self.unk_index = bos, pad, eos, unk
        self._symbols = dict(symbols) if symbols else {}
        self._tokenizer = tokenizer

    def __len__(self):
        return self._n

    def bos(self):
        return self.bos_index

    def pad(self):
        return self.pad_index

    def eos(self):
        return self.eos_index

    def unk(self):
        return self.unk_index

    def _lookup(self, sym):
        if sym in self._symbols:
            return int(self._symbols[sym])
        if self._tokenizer is not None:
            i = self._tokenizer.token_to_id(sym)
            if i is not None:
                return int(i)
        return None

    def resolves(self, sym) -> bool:
        return self._lookup(sym) is not None

    def index(self, sym):
        """Id of a textual symbol, unk if it is not in the table
        (metaseq/data/dictionary.py:67-72)."""
        i = self._lookup(sym)
        return self.unk_index if i is None else i
