"""Pragma grammar (behaviour of the reference parser, appy/utils.py:97-150)."""
import pytest

from appy_amd.frontend.pragma import format_pragma, parse_pragma


def test_parallel_for_simd():
    p = parse_pragma("#pragma parallel for simd")
    assert list(p.items()) == [("parallel_for", True), ("simd", True)]


def test_shared_is_always_a_list():
    assert parse_pragma("#pragma parallel for shared(s)")["shared"] == ["s"]
    assert parse_pragma("#pragma parallel for simd shared(sum, step)")["shared"] == ["sum", "step"]
    assert parse_pragma("#pragma parallel for to(a,b) from(c)")["to"] == ["a", "b"]


def test_other_clauses_string_or_tuple():
    assert parse_pragma("#pragma simd block(128)")["block"] == "128"
    assert parse_pragma("#pragma parallel for reduction(+:s)")["reduction"] == "+:s"
    assert parse_pragma("#pragma parallel for reduction(+:s, max:m)")["reduction"] == ("+:s", "max:m")


def test_unknown_clause_names_the_clause():
    with pytest.raises(ValueError) as e:
        parse_pragma("#pragma parallel for simd my_directive")
    assert "my_directive" in str(e.value)


def test_parallel_without_for_is_unknown():
    with pytest.raises(ValueError) as e:
        parse_pragma("#pragma parallel simd")
    assert "parallel" in str(e.value)


def test_unexpected_syntax():
    with pytest.raises(ValueError):
        parse_pragma("#pragma parallel for @@")


def test_round_trip():
    text = "#pragma parallel for simd shared(a, b)"
    assert parse_pragma(format_pragma(parse_pragma(text))) == parse_pragma(text)
