"""Tokenizers of Llama2.jl (src/tokenizer.jl), host side.  Token ids are 0-based here."""


class Tokenizer:
    pass


class BPETokenizer(Tokenizer):
    """src/tokenizer.jl:3-9.  id_to_token holds `bytes` (tokens may be partial UTF-8)."""

    def __init__(self, id_to_token, token_scores, bos_token_id, eos_token_id):
        self.id_to_token = [t if isinstance(t, bytes) else t.encode("utf-8") for t in id_to_token]
        self.token_to_id = {}
        for i, t in enumerate(self.id_to_token):  # later duplicates win, as Dict construction does
            self.token_to_id[t] = i
        self.token_scores = list(token_scores)
        self.bos_token_id = bos_token_id
        self.eos_token_id = eos_token_id

    def decode(self, ids):
        return b"".join(self.id_to_token[i] for i in ids).decode("utf-8", errors="replace")


def encode(text, tokenizer, pad_input=True):
    """encode(text, tokenizer) (src/tokenizer.jl:11-57 for BPE, :82-84 for characters)."""
    if isinstance(tokenizer, CharTokenizer):
        return [tokenizer.token_to_id[ch] for ch in text]
    data = text.encode("utf-8") if isinstance(text, str) else bytes(text)
    tokens = []
    if len(data) == 0:
        return tokens  # :16-18
    t2i, i2t, scores = tokenizer.token_to_id, tokenizer.id_to_token, tokenizer.token_scores
    if pad_input:
        tokens.append(t2i[b" "])  # :20-22
    for b in data:  # one token per code unit (:25-27)
        tokens.append(t2i[bytes([b])])
    while True:  # greedy merge of the best-scoring adjacent pair (:29-54)
        best_score, best_id, best_idx = float("-inf"), -1, -1
        for i in range(len(tokens) - 1):
            tid = t2i.get(i2t[tokens[i]] + i2t[tokens[i + 1]])
            if tid is not None and scores[tid] > best_score:
                best_score, best_id, best_idx = scores[tid], tid, i
        if best_idx == -1:
            break
        tokens[best_idx] = best_id
        del tokens[best_idx + 1]
    return tokens


class CharTokenizer(Tokenizer):
    """src/tokenizer.jl:59-80: sorted distinct characters, then "<s>" and "</s>"."""

    def __init__(self, text):
        self.id_to_token = sorted(set(text)) + ["<s>", "</s>"]
        self.token_to_id = {t: i for i, t in enumerate(self.id_to_token)}
        self.bos_token_id = len(self.id_to_token) - 2
        self.eos_token_id = len(self.id_to_token) - 1

    def decode(self, ids):
        return "".join(self.id_to_token[i] for i in ids)


def token_bytes(tokenizer, i):
    t = tokenizer.id_to_token[i]
    return t if isinstance(t, bytes) else t.encode("utf-8")
