"""Minimal symbol table with the reference's special-symbol layout
(metaseq/data/dictionary.py:22-42: <s>=0, <pad>=1, </s>=2, <unk>=3), enough for the
generator's constructor, which only asks for pad/unk/eos ids and the vocabulary size."""


class Dictionary:
    def __init__(self, vocab_size: int, bos=0, pad=1, eos=2, unk=3):
        self._n = int(vocab_size)
        self.bos_index, self.pad_index, self.eos_index, self.unk_index = bos, pad, eos, unk

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

    def index(self, sym):
        """Ids of textual symbols are unknown without a tokenizer file: everything maps to unk."""
        return self.unk_index
