"""The word machine (host C++, no GPU): tokenising, literals, user words,
list macro, hash builtins, base words, error handling.  Expected behaviour is
the language definition the reference machine implements
(blackriver/dag.cpp:43-556); each case states the rule it checks."""
import pytest

from blackriver_amd import host


@pytest.fixture()
def env(runtime):
    e = host.Env(3)
    yield e
    e.close()


def result(env, text):
    env.stack_clear()
    env.execute(text)
    out = []
    while env.stack_size:
        out.append(env.pop_number())
    return out[::-1]


def test_numbers_and_arithmetic(env):
    # a o b is evaluated as (second) o (top)
    assert result(env, "7 2 -") == [5]
    assert result(env, "7 2 /") == [3.5]
    assert result(env, "7 2 //") == [3]
    assert result(env, "-7 2 //") == [-3]          # (int) truncates toward zero
    assert result(env, "3 4 * 5 +") == [17]
    # '.' or 'e' makes a double, otherwise an integer
    assert result(env, "1e-05 2.5 10") == [1e-05, 2.5, 10]
    assert result(env, "-3 -2.5") == [-3, -2.5]


def test_separators_comments_and_grouping(env):
    # ( ) { } are whitespace; ; starts a comment; tabs count as blanks here
    assert result(env, "(1 2 +) {3 *} ; 100 +\n 4 +\t1 +") == [14]
    # a ';' inside a string is not a comment
    env.execute("'a;b' 's' !")
    assert env.stack_size == 0


def test_literals_ture_false_null_and_dollar_strings(env):
    assert result(env, "ture false true") == [1, 0, 1]
    # $name is a string that keeps its '$': it works as a hash key directly
    env.execute("42 $answer !")
    assert env.number("$answer") == 42
    assert result(env, "$answer @") == [42]
    # null is the empty string
    env.execute("null 'x' | 'k' !  7 'x' !")
    assert result(env, "'k' @ @") == [7]


def test_stack_words(env):
    assert result(env, "1 2 swap") == [2, 1]
    assert result(env, "1 2 3 rot") == [2, 3, 1]
    assert result(env, "5 dup") == [5, 5]
    assert result(env, "1 2 3 drop") == [1, 2]
    # dup2 leaves the pair three times
    assert result(env, "1 2 dup2") == [1, 2, 1, 2, 1, 2]


def test_list_macro_pushes_items_then_count(env):
    assert result(env, "[ 4 5 6 ]") == [4, 5, 6, 3]
    assert result(env, "[ ]") == [0]
    assert result(env, "9 [ 1 2 + ]") == [9, 3, 3]   # counts tokens, not values


def test_user_words_and_inlining(env):
    env.execute("%def sq dup * %end  %def quad sq sq %end")
    assert result(env, "3 quad") == [81]
    # a definition is visible to later compilations in the same environment
    assert result(env, "2 sq") == [4]
    assert env.disassemble("3 quad") == ["N:3", "W:dup", "W:*", "W:dup", "W:*"]


def test_hash_builtins_and_namespaces(env):
    env.execute("1 'a' !   1 #  2 'a' !   0 #")
    assert result(env, "'a' @") == [1]
    assert result(env, "1 # 'a' @ ## 0 #") == [2, 1]
    env.execute("'a' !!")
    with pytest.raises(host.HostError, match="Can't find value"):
        env.execute("'a' @")
    with pytest.raises(host.HostError, match="hash out"):
        env.execute("7 #")


def test_string_concat_order(env):
    env.execute("'ab' 'cd' | 'k' !  9 'abcd' !")
    assert result(env, "'k' @ @") == [9]


@pytest.mark.parametrize("text,msg", [
    ("nosuchword", "invalid symbol"),
    ("%def 1abc %end", "valid name"),
    ("%def dup %end", "valid name"),              # native words cannot be redefined
    ("%def a %def b %end %end", "inside another"),
    ("%end", "without"),
    ("%def a 1", "without #end"),
    ("[ 1 2", "without ']'"),
    ("1 ]", "without begin"),
    ("'abc", "string must end"),
    ("ab'cd'", "tokenize_line"),
    ("1 'x' +", "convert to number"),
    ("drop", "empty stack"),
])
def test_errors_are_reported_not_swallowed(env, text, msg):
    with pytest.raises(host.HostError, match=msg):
        env.execute(text)


def test_user_word_cannot_be_redefined(env):
    env.execute("%def once 1 %end")
    with pytest.raises(host.HostError, match="valid name"):
        env.execute("%def once 2 %end")


def test_cpu_tensors_views_and_storage_ops(env):
    env.execute("2048 1 'cpu' 'float' op.create 't' !   't' @ 2.5 op.fill")
    assert env.info("t")[2] == (2048,) and not env.info("t")[1]
    assert (env.read("t") == 2.5).all()
    # view with one dynamic (0) dimension: whatever fits after the offset
    env.execute("'t' @ 1024 0 256 2 op.view 'v' !  'v' @ op.zero")
    assert env.info("v")[2] == (4, 256)
    t = env.read("t")
    assert (t[:1024] == 2.5).all() and (t[1024:] == 0).all()
    assert env.info("v")[3] - env.info("t")[3] == 1024 * 4
    with pytest.raises(host.HostError, match="view out of shape"):
        env.execute("'t' @ 2000 100 1 op.view")
    with pytest.raises(host.HostError, match="one zero shape"):
        env.execute("'t' @ 0 0 0 2 op.view")
    # the host arena hands out whole pages only
    with pytest.raises(host.HostError, match="page"):
        env.execute("100 1 'cpu' 'float' op.create")
    # int tensors, copy between cpu tensors
    env.execute("1024 1 'cpu' 'int' op.create 'i' !  1024 1 'cpu' 'float' op.create 'u' !")
    env.execute("'u' @ 'v' @ op.copy")
    assert (env.read("u") == 0).all()
    with pytest.raises(host.HostError, match="same size"):
        env.execute("'u' @ 't' @ op.copy")


def test_cpu_tensors_have_no_math(env):
    env.execute("1024 1 'cpu' 'float' op.create 'a' !  1024 1 'cpu' 'float' op.create 'b' !")
    with pytest.raises(host.HostError, match="gelu|attn"):
        env.execute("'a' @ 'b' @ op.gelu")
    with pytest.raises(host.HostError, match="add"):
        env.execute("'a' @ 'b' @ 'a' @ op.add")


def test_load_and_save_roundtrip(env, tmp_path):
    import numpy as np
    x = np.arange(2048, dtype=np.float32)
    p = tmp_path / "x.bin"
    x.tofile(p)
    env.execute("2048 1 'cpu' 'float' op.create 'x' !  'x' @ '%s' io.load" % p)
    assert np.array_equal(env.read("x"), x)
    q = tmp_path / "y.bin"
    env.execute("'x' @ '%s' io.save" % q)
    assert np.array_equal(np.fromfile(q, dtype=np.float32), x)


def test_single_process_transport_shims(env):
    env.execute("1024 1 'cpu' 'float' op.create 'm' !  'm' @ 3 op.fill")
    env.execute("'m' @ 0 io.mpi.bcast")                     # rank 0 broadcasting to itself
    assert (env.read("m") == 3).all()
    with pytest.raises(host.HostError, match="mpi_recv"):   # nothing was sent
        env.execute("'m' @ 1 io.mpi.recv")


def test_fusion_pass_rewrites_only_push_separated_sequences(env):
    """`op.add op.add op.softmax` with nothing but operand pushes in between
    becomes two skipped words and the fused word; anything else is untouched,
    and the plain listing never changes."""
    seq = "'s' @ 'a' @ 's' @ op.add  's' @ 'm' @ 's' @ op.add  's' @ 'p' @ op.softmax"
    plain = env.disassemble(seq)
    fused = env.disassemble(seq, fused=True)
    assert [x for x in plain if x.startswith("W:")] == ["W:op.add", "W:op.add", "W:op.softmax"]
    assert [x for x in fused if x[0] in "W-"] == ["-:op.add", "-:op.add", "W:op.add_add_softmax"]
    assert [x for x in fused if x[0] not in "W-"] == [x for x in plain if x[0] != "W"]
    # a number push, a hash switch or another word in between breaks the pattern
    for middle in ("1 drop", "0 #", "op.sync"):
        broken = seq.replace("op.add  's' @ 'm'", "op.add " + middle + " 's' @ 'm'", 1)
        assert env.disassemble(broken, fused=True) == env.disassemble(broken)
    # two sequences in one program are both rewritten
    assert env.disassemble(seq + " " + seq, fused=True).count("W:op.add_add_softmax") == 2
    # a lone add followed by softmax is not a match
    short = "'s' @ 'm' @ 's' @ op.add  's' @ 'p' @ op.softmax"
    assert env.disassemble(short, fused=True) == env.disassemble(short)


def test_fusion_pass_folds_a_trailing_copy_into_the_producer(env):
    """`op.layernorm op.copy` and the score softmax followed by `op.copy`
    become one word each; the four-word pattern wins over the three-word one,
    which still applies when no copy follows."""
    ln = "'x' @ 'mean' @ 'var' @ 'g' @ 'b' @ 'y' @ 1e-5 op.layernorm  'y.h' @ 'y' @ op.copy"
    fused = env.disassemble(ln, fused=True)
    assert [x for x in fused if x[0] in "W-"] == ["-:op.layernorm", "W:op.layernorm_copy"]
    sm = "'s' @ 'a' @ 's' @ op.add  's' @ 'm' @ 's' @ op.add  's' @ 's' @ op.softmax"
    with_copy = env.disassemble(sm + "  's.h' @ 's' @ op.copy", fused=True)
    assert [x for x in with_copy if x[0] in "W-"] == ["-:op.add", "-:op.add", "-:op.softmax",
                                                      "W:op.add_add_softmax_copy"]
    both = env.disassemble(sm + "  's.h' @ 's' @ op.copy  " + sm + " op.sync 's.h' @ 's' @ op.copy", fused=True)
    assert [x for x in both if x.startswith("W:")] == ["W:op.add_add_softmax_copy", "W:op.add_add_softmax",
                                                       "W:op.sync", "W:op.copy"]
