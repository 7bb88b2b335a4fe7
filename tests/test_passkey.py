"""CPU: the prompt of the pass key retrieval run (tiny-gemma_amd/host/passkey.hpp, counterpart of the reference's
tests/passkey.cpp:10-54) against a statement of the same text by slicing, and the two random draws."""
import ctypes as C
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "tests", "host", "libtokenizer_shim.so")

TASK = ("There is an important info hidden inside a lot of irrelevant text. Find it and memorize them. "
        "I will quiz you about the important information there. ")
FILLER = "The grass is green. The sky is blue. The sun is yellow. Here we go. There and back again. "
QUESTION = "\nWhat is the pass key? The pass key is"


def shim():
    if not os.path.exists(SHIM):
        pytest.fail("tests/host/libtokenizer_shim.so is not built: run __graft_entry__.build()")
    L = C.CDLL(SHIM)
    L.passkey_prompt.argtypes = [C.c_int, C.c_int, C.c_int, C.c_char_p, C.c_int]
    L.passkey_draw.argtypes = [C.c_uint, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.passkey_draw.restype = None
    return L


def built_prompt(L, n_garbage, prefix, key):
    cap = n_garbage + 4096
    buf = C.create_string_buffer(cap)
    n = L.passkey_prompt(n_garbage, prefix, key, buf, cap)
    assert 0 < n <= cap
    return buf.raw[:n].decode()


def expected_prompt(n_garbage, prefix, key):
    """passkey.cpp:22-50: the filler in front of the number is the first `prefix` characters of the repeated block;
    behind it come (n_garbage - prefix) // 90 whole blocks and then prefix % 90 characters (the reference reuses
    the prefix's remainder there)."""
    front = (FILLER * (prefix // len(FILLER) + 1))[:prefix]
    back = FILLER * ((n_garbage - prefix) // len(FILLER)) + FILLER[:prefix % len(FILLER)]
    line = "\nThe pass key is %d. Remember it. %d is the pass key.\n" % (key, key)
    return TASK + front + line + back + QUESTION


def draw(L, seed, n_garbage):
    p, k = C.c_int(), C.c_int()
    L.passkey_draw(seed, n_garbage, C.byref(p), C.byref(k))
    return p.value, k.value


@pytest.mark.parametrize("n_garbage,prefix,key", [(1, 1, 1), (89, 45, 7), (90, 90, 50000), (91, 1, 123), (1000, 333, 31337),
                                                  (20000, 19999, 4242), (20000, 90, 9), (5000, 2500, 50000)])
def test_prompt_text(n_garbage, prefix, key):
    assert len(FILLER) == 90
    L = shim()
    got = built_prompt(L, n_garbage, prefix, key)
    assert got == expected_prompt(n_garbage, prefix, key)
    assert got.count(str(key) + " is the pass key.") == 1 and got.startswith(TASK) and got.endswith(QUESTION)
    # the number sits exactly `prefix` characters behind the task description
    assert got.index("\nThe pass key is ") == len(TASK) + prefix


def test_draws_are_repeatable_and_in_range():
    L = shim()
    seen = set()
    for seed in range(200):
        p, k = draw(L, seed, 777)
        assert (p, k) == draw(L, seed, 777)
        assert 1 <= p <= 777 and 1 <= k <= 50000
        seen.add((p, k))
    assert len(seen) > 190
    # n_garbage 1 leaves one place for the number
    assert draw(L, 5, 1)[0] == 1
