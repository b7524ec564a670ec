"""The text wrapper (tokenizer.py) and the command line's handling of text prompts, without a GPU.  The
vocabulary is a small word-level one written here; what a real vocabulary does with text is the
`tokenizers` package's business, not this wrapper's."""
import json
import os

import pytest

tokenizers = pytest.importorskip("tokenizers")

WORDS = ["[UNK]", "<eos>", "the", "capital", "of", "france", "is", "paris", "a", "city"]


def write_tokenizer(path):
    from tokenizers import Tokenizer, models, normalizers, pre_tokenizers
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(WORDS)}, unk_token="[UNK]"))
    tok.normalizer = normalizers.Lowercase()
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.add_special_tokens(["<eos>"])
    tok.save(str(path))
    return str(path)


def test_tokenize_text_and_pieces(tmp_path):
    from mini_llm_runtime_amd.tokenizer import Tokenizer
    write_tokenizer(tmp_path / "tokenizer.json")
    for where in (tmp_path, tmp_path / "tokenizer.json"):             # the folder or the file
        tok = Tokenizer(str(where), expected_vocabulary=16, eog_ids=(1,))
        assert tok.vocabulary_size() == len(WORDS)
        assert tok.tokenize("The capital of France is") == [2, 3, 4, 5, 6]
        assert tok.tokenize("Paris is a town") == [7, 6, 8, 0]
        assert tok.tokenize("paris <eos>") == [7, 1]                    # a special token written out is taken as such
        assert tok.text([7, 6, 8, 9]) == "paris is a city"
        assert tok.text([7, 1]) == "paris" and tok.token_piece(1) == "" and tok.token_piece(9) == "city"
        assert tok.is_eog(1) and not tok.is_eog(7)


def test_the_vocabulary_must_fit_the_embedding_matrix(tmp_path):
    from mini_llm_runtime_amd.tokenizer import Tokenizer, TokenizerError
    write_tokenizer(tmp_path / "tokenizer.json")
    Tokenizer(str(tmp_path), expected_vocabulary=len(WORDS))             # exactly as many rows: fits
    with pytest.raises(TokenizerError, match="does not fit the embedding matrix"):
        Tokenizer(str(tmp_path), expected_vocabulary=len(WORDS) - 1)


def test_errors_name_what_is_wrong(tmp_path):
    from mini_llm_runtime_amd.tokenizer import MAX_PROMPT_BYTES, Tokenizer, TokenizerError
    with pytest.raises(TokenizerError, match="no tokenizer.json"):
        Tokenizer(str(tmp_path), 16)
    (tmp_path / "broken").mkdir()
    (tmp_path / "broken" / "tokenizer.json").write_text("{ not json")
    with pytest.raises(TokenizerError, match="cannot load the tokenizer"):
        Tokenizer(str(tmp_path / "broken"), 16)
    tok = Tokenizer(write_tokenizer(tmp_path / "tokenizer.json"), 16)
    with pytest.raises(TokenizerError, match="256 KiB"):
        tok.tokenize("a " * (MAX_PROMPT_BYTES // 2 + 1))
    assert len(tok.tokenize("a " * 1000)) == 1000


def test_command_line_refuses_text_without_a_vocabulary_before_it_reads_weights(tmp_path, capsys):
    """Option handling only: nothing here reaches the GPU (the folder holds no weights at all)."""
    from mini_llm_runtime_amd.cli import main
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps({"architectures": ["Qwen3ForCausalLM"]}))
    for args, text in [(["--model", str(folder), "--prompt", "hello"], "no tokenizer.json"),
                       (["--model", str(folder)], "no tokenizer.json"),
                       (["--model", str(folder), "--prompt-ids", "1", "--tokenizer", str(tmp_path / "none")],
                        "no tokenizer.json there"),
                       (["--model", str(folder), "--prompt", "hello", "--prompt-ids", "1"], "one of them"),
                       (["--model", str(folder), "--prompt", "hello", "--prompts-file", "x"], "one of them")]:
        assert main(args) == 1
        assert text in capsys.readouterr().err, args
