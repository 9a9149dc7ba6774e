"""Transcribes the reference's 6-sentence WordPiece known-answer test into a JSON fixture.

The reference test file is read AS TEXT (nothing from it is imported or executed):
python/cudf/cudf/tests/text/test_subword_tokenizer.py holds six input sentences
and the expected token ids for max_words in {0, 200} and for max_words == 10;
python/cudf/cudf/tests/data/text/vocab.txt is the 3500-entry vocabulary (a data file).
Run once in the authoring container:  python tests/golden/transcribe_subword_fixture.py
"""
import ast
import json
import os
import shutil

REF = "/root/reference/python/cudf/cudf/tests"
HERE = os.path.dirname(os.path.abspath(__file__))


def series_lists(node):
    """[[ints], ...] from a `cudf.Series([cudf.Series([...], dtype=...), ...])` AST node."""
    out = []
    for inner in node.args[0].elts:
        out.append([ast.literal_eval(e) for e in inner.args[0].elts])
    return out


def main():
    src = open(os.path.join(REF, "text", "test_subword_tokenizer.py")).read()
    tree = ast.parse(src)
    fn = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == "test_text_wordpiece_tokenize")
    sentences, expected_all, expected_10 = None, None, None
    for node in ast.walk(fn):
        if isinstance(node, ast.Assign) and isinstance(node.targets[0], ast.Name):
            name = node.targets[0].id
            if name == "s":
                sentences = [ast.literal_eval(e) for e in node.value.args[0].elts]
            elif name == "expected":
                lists = series_lists(node.value)
                if expected_all is None:
                    expected_all = lists
                else:
                    expected_10 = lists
    assert len(sentences) == 6 and len(expected_all) == 6 and len(expected_10) == 6
    shutil.copyfile(os.path.join(REF, "data", "text", "vocab.txt"), os.path.join(HERE, "bert_vocab_3500.txt"))
    fixture = {
        "source": "python/cudf/cudf/tests/text/test_subword_tokenizer.py:17-…; vocab python/cudf/cudf/tests/data/text/vocab.txt",
        "vocab_file": "bert_vocab_3500.txt",
        "rows": sentences,
        "expected": {"0": expected_all, "200": expected_all, "10": expected_10},
    }
    with open(os.path.join(HERE, "wordpiece_bert_sentences.json"), "w") as f:
        json.dump(fixture, f, indent=1, ensure_ascii=False)
    print("rows", [len(s.encode()) for s in sentences], "tokens", [len(e) for e in expected_all])


if __name__ == "__main__":
    main()
