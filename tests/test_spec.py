"""The model-free half of speculative decoding: the prompt-lookup drafter against the reference's
own known answers (cera/src/spec.rs:273-318).  Runs through the backend library's C face, which
loads without a GPU."""
from cera_amd import llama_api as L


def test_draft_predicts_repeated_continuation():
    toks = [10, 20, 30, 10, 20]
    assert L.prompt_lookup_draft(toks, 2, 3) == [30, 10, 20]
    assert L.prompt_lookup_draft(toks, 2, 1) == [30]          # k bounds the draft length


def test_draft_uses_most_recent_match():
    assert L.prompt_lookup_draft([7, 8, 9, 7, 8, 7, 8], 2, 2) == [7, 8]


def test_draft_empty_when_no_match_or_degenerate():
    assert L.prompt_lookup_draft([1, 2, 3, 4, 5], 2, 3) == []
    assert L.prompt_lookup_draft([1, 2, 3], 0, 3) == []
    assert L.prompt_lookup_draft([1, 2, 3], 2, 0) == []
    assert L.prompt_lookup_draft([1, 2], 2, 3) == []            # len == ngram
    assert L.prompt_lookup_draft([], 2, 3) == []


def test_draft_respects_sequence_end():
    assert L.prompt_lookup_draft([1, 2, 9, 5, 1, 2], 2, 5) == [9, 5, 1, 2]
