"""scala/TensorDslHIP.scala is source for the Lantern tree and is not compiled here (no JVM): this test reads it as text.
Every `Backend` trait method (TensorDifferentiation.scala:137-379) is overridden, and every library call it emits, all
through the one helper hip("lh_name", args...), names a function of include/lantern_hip.h with that function's argument
count.  Calls written as literal C text ("lh_malloc(" in the code generator) are checked by name."""
import os
import re

from tests.test_trait_names import TRAIT_METHODS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SCALA = os.path.join(ROOT, "scala", "TensorDslHIP.scala")
HEADER = os.path.join(ROOT, "include", "lantern_hip.h")


def _split_top_level(text):
    """Comma-separated pieces of `text`, commas inside brackets and string literals not counted."""
    parts, depth, cur, i, in_str = [], 0, [], 0, False
    while i < len(text):
        ch = text[i]
        if in_str:
            cur.append(ch)
            if ch == "\\":
                cur.append(text[i + 1]); i += 1
            elif ch == '"':
                in_str = False
        elif ch == '"':
            in_str = True; cur.append(ch)
        elif ch in "([{":
            depth += 1; cur.append(ch)
        elif ch in ")]}":
            depth -= 1; cur.append(ch)
        elif ch == "," and depth == 0:
            parts.append("".join(cur).strip()); cur = []
        else:
            cur.append(ch)
        i += 1
    tail = "".join(cur).strip()
    if tail:
        parts.append(tail)
    return parts


def _matching_paren(text, open_at):
    depth, i, in_str = 0, open_at, False
    while i < len(text):
        ch = text[i]
        if in_str:
            if ch == "\\":
                i += 1
            elif ch == '"':
                in_str = False
        elif ch == '"':
            in_str = True
        elif ch == "(":
            depth += 1
        elif ch == ")":
            depth -= 1
            if depth == 0:
                return i
        i += 1
    raise AssertionError("unbalanced parenthesis at offset %d" % open_at)


def header_arity():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(lh_[a-z0-9_]+)\s*\(", text):
        close = _matching_paren(text, m.end() - 1)
        args = text[m.end():close].strip()
        out[m.group(1)] = 0 if args in ("", "void") else len(_split_top_level(args))
    return out


def scala_source():
    text = open(SCALA).read()
    return re.sub(r"//[^\n]*", "", text)      # line comments may mention calls loosely; only code is checked


def scala_calls():
    """[(name, argument count, line)] for every hip("lh_...", ...) in the Scala source."""
    text = scala_source()
    calls = []
    for m in re.finditer(r'\bhip\(\s*"(lh_[a-z0-9_]+)"', text):
        open_at = text.index("(", m.start())
        close = _matching_paren(text, open_at)
        pieces = _split_top_level(text[open_at + 1:close])
        calls.append((m.group(1), len(pieces) - 1, text.count("\n", 0, m.start()) + 1))
    return calls


def test_every_trait_method_is_overridden():
    text = scala_source()
    defined = set(re.findall(r"\boverride\s+def\s+([A-Za-z0-9_]+)", text))
    missing = [m for m in TRAIT_METHODS if m not in defined]
    assert not missing, "trait methods without an override in BackendHIP: %s" % missing


def test_every_emitted_call_matches_the_header():
    arity = header_arity()
    calls = scala_calls()
    assert len(calls) >= 75
    unknown = sorted({(n, line) for n, _, line in calls if n not in arity})
    assert not unknown, "calls to functions the header does not declare: %s" % unknown
    wrong = [(n, got, arity[n], line) for n, got, line in calls if got != arity[n]]
    assert not wrong, "(name, arguments passed, arguments declared, line): %s" % wrong


def test_literal_c_text_names_declared_functions():
    """Names inside string literals (the code generator's lh_malloc / lh_h2d lines, unchecked("(long)lh_mark()"))."""
    arity = header_arity()
    names = set(re.findall(r"\b(lh_[a-z0-9_]+)\b", scala_source()))
    assert names - set(arity) == set(), sorted(names - set(arity))


# Declared operators the Scala backend has no call for, with the reason.  Everything else it does not call must be runtime
# plumbing (error mode, events, pinned memory, capture, tuning switches), which generated programs reach by name if at all.
NOT_CALLED = {
    # fused forms: the backend emits the trait's one call per method, and the LIBRARY runs these when it recognises the chain
    # (conv -> batchNorm -> [+] -> relu in place, their gradients, runs of optimizer calls); they stay callable for hand-written hosts
    "lh_add_relu", "lh_add_relu_grad", "lh_bn_apply", "lh_bn_apply_add_relu", "lh_bn_bwd_add_relu", "lh_bn_bwd_relu", "lh_bn_stats",
    "lh_bn_train_fwd_relu", "lh_conv2d_fwd_bnstats", "lh_conv2d_fwd_bn_apply", "lh_concat_grad_beta", "lh_multi_momentum", "lh_multi_sgd",
    # outputs the backend allocates come from lh_malloc (zero-filled, cleared on demand): the uncleared form is for hand-written hosts
    # (the code generator still emits it for literal arrays it uploads at once)
    # superseded within the trait mapping: padded average pooling covers pad 0; the dense max-pool gradient replaces the scatter form
    "lh_avgpool_fwd", "lh_avgpool_bwd", "lh_maxpool_bwd",
    # the zero-state forms: the backend always calls the *_init forms, with NULL for a state it was not given
    "lh_rnn_fwd", "lh_rnn_bwd", "lh_rnn_gated_fwd", "lh_rnn_gated_bwd",
    # the reserve size is a staging-time product in Scala (same formula, checked in tests/test_parity_ops.py against the call)
    "lh_rnn_gated_reserve_floats",
    # data loader side, not the trait
    "lh_cifar_decode",
}
PLUMBING = re.compile(r"^lh_(set_|get_|last_error|clear_error|sync|heap_|free_top|host_|h2d_async|d2h_async|copy_join|capture_|graph_|tune_|"
                      r"side_forks|side_join|event_|prof_|cmdlist_|multi_momentum_static|flush_deferred|fusion_stats|work_collect)")


def test_the_backend_uses_the_whole_operator_surface():
    used = set(re.findall(r"\b(lh_[a-z0-9_]+)\b", scala_source()))
    unused = set(header_arity()) - used
    unexplained = sorted(n for n in unused if n not in NOT_CALLED and not PLUMBING.match(n))
    assert not unexplained, unexplained
    assert NOT_CALLED <= unused, sorted(NOT_CALLED - unused)
