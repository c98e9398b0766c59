"""A tiny ``tokenizer.json`` for the tests of the text path, built with the ``tokenizers`` library: a
word-level vocabulary of a few words, and the Llama 3 special tokens as added special tokens behind it."""

WORDS = ["<unk>", "hello", "world", "be", "brief", "system", "user", "assistant", "ipython", "<|", "|>", "eot_id",
         "how", "are", "you", "fine", "thanks", "again", "begin_of_text", "tool"]
SPECIALS = ["<|begin_of_text|>", "<|start_header_id|>", "<|end_header_id|>", "<|eot_id|>"]
ID = {w: i for i, w in enumerate(WORDS + SPECIALS)}
BOS, START, END, EOT = (ID[s] for s in SPECIALS)


def write_tokenizer(folder) -> str:
    from tokenizers import AddedToken, Tokenizer, models, pre_tokenizers

    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(WORDS)}, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.add_special_tokens([AddedToken(s, special=True) for s in SPECIALS])
    path = str(folder / "tokenizer.json")
    tok.save(path)
    return path


def header(role: str):
    """What ``<|start_header_id|>role<|end_header_id|>\\n\\n`` must encode to (the line feeds are no tokens here)."""
    return [START, ID[role], END]
