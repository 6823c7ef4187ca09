"""The IR front end (triton_amd/ir.py): the reference's grammar (IrParser.py:13-134) and the recogniser that maps a
candidate onto a hand-written module.  The reference ships no IR files (its `evaluation/` inputs are git-ignored), so
the candidates here are written for this test in that grammar, with the child layouts the code generator expects
(TritonGen.py:2273-2281 loops, :2474-2480 load, :2573-2578 store): several structurally different programs per
workload, as equality saturation would produce them, plus programs that are not attention variants."""
import pytest

from triton_amd import ir

FULL2 = "(index (fulltile) (fulltile))"


def projections(x="(load (input X) (index fulltile fulltile))", fused=True):
    """Q1/K1/V1 [M,N] = x @ W*, column tiles of 64 in a parallel loop; one kernel or three."""
    def one(t, w):
        return f"(store (tensor {t}) (* {x} (load (input {w}) (index fulltile (tile n)))) (index fulltile (tile n)))"
    if fused:
        return "(ploop 0 N 64 n (seq " + " ".join(one(t, w) for t, w in (("Q1", "WQ"), ("K1", "WK"), ("V1", "WV"))) + "))"
    return " ".join(f"(ploop 0 N 64 n {one(t, w)})" for t, w in (("Q1", "WQ"), ("K1", "WK"), ("V1", "WV")))


def head_rows(t):
    return f"(permute3 (unsqueeze (load (tensor {t}) (index fulltile (tile h))) 1) 1 0 2)"


APPEND = ("(store (input K_cache) {k} (index (elem h) (const_tile P M) fulltile)) "
          "(store (input V_cache) " + head_rows("V1") + " (index (elem h) (const_tile P M) fulltile))")
SCORES = "(* {q} (permute3 (load (input K_cache) (index (elem h) (tile p) fulltile)) 0 2 1))"


def attention(q=None, k=None, divide_last=True, extra_in_loop="", extra_after="", scores_tensor=False):
    q = q or head_rows("Q1")
    k = k or head_rows("K1")
    s = SCORES.format(q=q)
    e = "(load (tensor C_exp) (index (elem h) fulltile (tile p)))"
    body = f"(store (tensor C_exp) (exp {s}) (index (elem h) fulltile (tile p))) "
    if scores_tensor:
        body = f"(store (tensor C) {s} (index (elem h) fulltile (tile p))) " \
               f"(store (tensor C_exp) (exp (load (tensor C) (index (elem h) fulltile (tile p)))) (index (elem h) fulltile (tile p))) "
    body += f"(store (tensor C_sum) (+ (load (tensor C_sum) (index (elem h) fulltile)) (rsum {e} 2)) (index (elem h) fulltile)) "
    v = "(load (input V_cache) (index (elem h) (tile p) fulltile))"
    if divide_last:
        body += f"(store (tensor O) (+ (load (tensor O) (index (elem h) fulltile fulltile)) (* {e} {v})) (index (elem h) fulltile fulltile)) "
        final = "(store (output O2) (squeeze (permute3 (/ (load (tensor O) (index (elem h) fulltile fulltile)) " \
                "(bcast (load (tensor C_sum) (index (elem h) fulltile)) 2)) 1 0 2) 1) (index fulltile (tile h)))"
        loop = f"(sloop 0 P+M 16 p (seq {body}{extra_in_loop}))"
        return f"(ploop 0 H 1 h (seq {APPEND.format(k=k)} {loop} {final} {extra_after}))"
    # normalise the probabilities first (a second pass over the keys), then multiply by V
    loop1 = f"(sloop 0 P+M 16 p (seq {body}))"
    p = f"(/ {e} (bcast (load (tensor C_sum) (index (elem h) fulltile)) 2))"
    body2 = f"(store (tensor C_div) {p} (index (elem h) fulltile (tile p))) " \
            f"(store (output O2) (+ (load (output O2) (index fulltile (tile h))) (squeeze (permute3 (* (load (tensor C_div) (index (elem h) fulltile (tile p))) {v}) 1 0 2) 1)) (index fulltile (tile h))) "
    loop2 = f"(sloop 0 P+M 16 p (seq {body2}{extra_in_loop}))"
    return f"(ploop 0 H 1 h (seq {APPEND.format(k=k)} {loop1} {loop2} {extra_after}))"


def rms(x, axis, n):
    """x / sqrt(mean(x^2)) in the IR's operators (no rsqrt node: NodeType.py lists sqrt and '/')."""
    return f"(/ {x} (bcast (sqrt (/ (rsum (sqr {x}) {axis}) {n})) {axis}))"


X = "(load (input X) (index fulltile fulltile))"
P_DIV = "(load (tensor C_div) (index (elem h) fulltile (tile p)))"
ROCO_STATS = (f"(store (output C_out1) (rsum {P_DIV} 1) (index (elem h) (tile p))) "
              f"(store (output C_out2) (rsum (sqr {P_DIV}) 1) (index (elem h) (tile p))) ")
KF_E = "(exp (/ (+ " + SCORES.format(q=head_rows("Q1")) + " (load (input noise) (index (elem h) fulltile (tile p)))) 1.5))"
KF_LOOP1 = (f"(store (tensor C_exp_perturb) {KF_E} (index (elem h) fulltile (tile p))) "
            "(store (tensor C_sum_perturb) (+ (load (tensor C_sum_perturb) (index (elem h) fulltile)) "
            "(rsum (load (tensor C_exp_perturb) (index (elem h) fulltile (tile p))) 2)) (index (elem h) fulltile)) ")
KF_OUT = ("(sloop 0 P+M 16 p (store (output C_out) (rsum (/ (load (tensor C_exp_perturb) (index (elem h) fulltile (tile p))) "
          "(bcast (load (tensor C_sum_perturb) (index (elem h) fulltile)) 2)) 1) (index (elem h) (tile p))))")

CANDIDATES = {
    "vanilla": [
        f"(seq {projections()} {attention()})",
        f"(seq {projections(fused=False)} {attention(divide_last=False)})",
        f"(seq {projections()} {attention(scores_tensor=True)})",
    ],
    "prenorm": [
        f"(seq (store (tensor X_norm) {rms(X, 1, 'N')} {FULL2}) "
        f"{projections(x='(load (tensor X_norm) (index fulltile fulltile))')} {attention()})",
        # the row scale applied after the projection: (x r) @ W = r (x @ W); the squaring written as x * x
        f"(seq (store (tensor X2) (sqrt (/ (rsum (x {X} {X}) 1) N)) (index fulltile)) "
        f"{projections()} "
        f"{attention(q='(/ ' + head_rows('Q1') + ' (bcast (load (tensor X2) (index fulltile)) 1))', k='(/ ' + head_rows('K1') + ' (bcast (load (tensor X2) (index fulltile)) 1))')})".replace(
            "(store (input V_cache) " + head_rows("V1"),
            "(store (input V_cache) (/ " + head_rows("V1") + " (bcast (load (tensor X2) (index fulltile)) 1))"),
    ],
    "qknorm": [
        f"(seq {projections()} {attention(q=rms(head_rows('Q1'), 2, 'D'), k=rms(head_rows('K1'), 2, 'D'))})",
        f"(seq {projections(fused=False)} {attention(q=rms(head_rows('Q1'), 2, 'D'), k=rms(head_rows('K1'), 2, 'D'), divide_last=False)})",
    ],
    "keyformer": [
        f"(seq {projections()} {attention(extra_in_loop=KF_LOOP1, extra_after=KF_OUT)})",
        f"(seq {projections(fused=False)} {attention(divide_last=False, extra_in_loop=KF_LOOP1, extra_after=KF_OUT)})",
    ],
    "roco": [
        f"(seq {projections()} {attention(divide_last=False, extra_in_loop=ROCO_STATS)})",
    ],
}
LINEAR = {
    # LoRA (lora_benchmark.py:41-53): X@W + (X@A)@B, fused and in three kernels through the driver's intermediates
    "lora": [
        "(ploop 0 P 64 p (store (output O) (+ (* (load (input X) (index fulltile fulltile)) (load (input W) (index fulltile (tile p)))) "
        "(* (* (load (input X) (index fulltile fulltile)) (load (input A) (index fulltile fulltile))) (load (input B) (index fulltile (tile p))))) (index fulltile (tile p))))",
        "(seq (ploop 0 R 16 r (store (tensor D) (* (load (input X) (index fulltile fulltile)) (load (input A) (index fulltile (tile r)))) (index fulltile (tile r)))) "
        "(ploop 0 P 64 p (seq (store (tensor C) (* (load (input X) (index fulltile fulltile)) (load (input W) (index fulltile (tile p)))) (index fulltile (tile p))) "
        "(store (tensor E) (* (load (tensor D) (index fulltile fulltile)) (load (input B) (index fulltile (tile p)))) (index fulltile (tile p))) "
        "(store (output O) (+ (load (tensor C) (index fulltile (tile p))) (load (tensor E) (index fulltile (tile p)))) (index fulltile (tile p))))))",
    ],
    # gated MLP (gmlp_benchmark.py:53-64), with the sigmoid operator and spelled out with exp
    "gmlp": [
        "(ploop 0 N 64 n (store (output O) (x (sigmoid (* (load (input X) (index fulltile fulltile)) (load (input W1) (index fulltile (tile n))))) "
        "(* (load (input X) (index fulltile fulltile)) (load (input W2) (index fulltile (tile n))))) (index fulltile (tile n))))",
        "(ploop 0 N 64 n (seq (store (tensor C1) (* (load (input X) (index fulltile fulltile)) (load (input W1) (index fulltile (tile n)))) (index fulltile (tile n))) "
        "(store (tensor C1_exp) (exp (- 0 (load (tensor C1) (index fulltile (tile n))))) (index fulltile (tile n))) "
        "(store (tensor C2) (* (load (input X) (index fulltile fulltile)) (load (input W2) (index fulltile (tile n)))) (index fulltile (tile n))) "
        "(store (output O) (/ (x (load (tensor C1) (index fulltile (tile n))) (load (tensor C2) (index fulltile (tile n)))) "
        "(+ 1 (load (tensor C1_exp) (index fulltile (tile n))))) (index fulltile (tile n)))))",
    ],
}
UNSUPPORTED = {
    "lora without the adapter": "(ploop 0 P 64 p (store (output O) (+ (* (load (input X) (index fulltile fulltile)) (load (input W) (index fulltile (tile p)))) "
                                "(+ (load (input A) (index fulltile fulltile)) (load (input B) (index fulltile (tile p))))) (index fulltile (tile p))))".replace("(+ (load (input A)", "(x (load (input A)"),
    "gated-MLP inputs without a gate": "(ploop 0 N 64 n (store (output O) (x (* (load (input X) (index fulltile fulltile)) (load (input W1) (index fulltile (tile n)))) "
                                       "(* (load (input X) (index fulltile fulltile)) (load (input W2) (index fulltile (tile n))))) (index fulltile (tile n))))",
    "unknown inputs": "(ploop 0 N 64 n (store (output O) (* (load (input X) (index fulltile fulltile)) (load (input Wz) (index fulltile (tile n)))) (index fulltile (tile n))))",
    "sigmoid on attention inputs": "(ploop 0 N 64 n (store (output O2) (x (sigmoid (* (load (input X) (index fulltile fulltile)) (load (input WQ) (index fulltile (tile n))))) "
            "(* (load (input X) (index fulltile fulltile)) (load (input WK) (index fulltile (tile n))))) (index fulltile (tile n))))",
    "projection only": f"(seq {projections()} (ploop 0 H 1 h (store (output O2) (load (tensor Q1) (index fulltile (tile h))) (index fulltile (tile h)))))",
    "no cache append": f"(seq {projections()} {attention()})".replace("(store (input K_cache)", "(store (tensor K_new)"),
    "prenorm and qknorm at once": f"(seq (store (tensor X_norm) {rms(X, 1, 'N')} {FULL2}) "
                                  f"{projections(x='(load (tensor X_norm) (index fulltile fulltile))')} "
                                  f"{attention(q=rms(head_rows('Q1'), 2, 'D'), k=rms(head_rows('K1'), 2, 'D'))})",
    "noise without C_out": f"(seq {projections()} {attention(extra_in_loop=KF_LOOP1)})",
    "roco with one statistic": f"(seq {projections()} {attention(divide_last=False, extra_in_loop=ROCO_STATS.split('(store (output C_out2)')[0])})",
}


@pytest.mark.parametrize("variant,index", [(v, i) for v, c in CANDIDATES.items() for i in range(len(c))])
def test_candidates_are_recognised(variant, index):
    m = ir.recognise(CANDIDATES[variant][index])
    assert m.variant == variant, m.reason


@pytest.mark.parametrize("variant,index", [(v, i) for v, c in LINEAR.items() for i in range(len(c))])
def test_lora_and_gated_mlp_candidates_are_recognised(variant, index):
    m = ir.recognise(LINEAR[variant][index])
    assert m.variant == variant, m.reason
    if variant == "gmlp":
        # the first candidate gates with sigmoid(X W1); the second computes C1 C2 / (1 + exp(-C1)) = SiLU(C1) C2
        assert m.kwargs == {"gate": ("sigmoid", "silu")[index]}
    else:
        assert m.kwargs == {}


def test_keyformer_temperature_is_read_off_the_candidate():
    """The module is built with the divisor the candidate applies to its perturbed scores (ref_rms.py:172 divides by
    1.5); a candidate with another constant gets that one, one without a division gets 1, and a divisor that is not a
    number is not something the hand-written module can be built for."""
    c = CANDIDATES["keyformer"][0]
    assert ir.recognise(c).kwargs == {"tau": 1.5}
    assert ir.recognise(c.replace("noise) (index (elem h) fulltile (tile p)))) 1.5))", "noise) (index (elem h) fulltile (tile p)))) 2))")).kwargs == {"tau": 2.0}
    no_div = c.replace("(exp (/ (+ ", "(exp (+ ").replace("(load (input noise) (index (elem h) fulltile (tile p)))) 1.5))", "(load (input noise) (index (elem h) fulltile (tile p)))))")
    m = ir.recognise(no_div)
    assert m.variant == "keyformer" and m.kwargs == {"tau": 1.0}, m.reason
    m = ir.recognise(c.replace("(tile p)))) 1.5))", "(tile p)))) T))"))
    assert not m and "temperature" in m.reason


def _tree(n):
    """ir.Node -> nested tuples, so that the expected trees below can be written as plain literals."""
    return (n.op, *(_tree(a) for a in n.args)) if isinstance(n, ir.Node) else n


def test_parse_against_trees_written_out_by_hand_from_the_reference_parser():
    """What IrParser.parse builds for the constructs that have code of their own there, written out by hand
    (a VAR child of the reference is a bare string here, a NUM child an int, other nodes (op, children...))."""
    # names under input / output / tensor: a comma-separated list becomes one VAR child per name, in order
    # (IrParser.py:63-87); spaces around the commas do not matter (the tokenizer splits on them, :13-19)
    assert _tree(ir.parse("(input X,Y)")) == ("input", "X", "Y")
    assert _tree(ir.parse("(output A , B)")) == ("output", "A", "B")
    assert _tree(ir.parse("(tensor C_exp, C_sum ,C_div)")) == ("tensor", "C_exp", "C_sum", "C_div")
    # a single name is parsed as an ordinary expression: one VAR child (IrParser.py:88-91)
    assert _tree(ir.parse("(input X)")) == ("input", "X")
    # `fulltile` and `dummy` are nodes without children whether bare (IrParser.py:44-49) or parenthesised (:107, :123)
    assert _tree(ir.parse("(index fulltile (fulltile) (tile n))")) == ("index", ("fulltile",), ("fulltile",), ("tile", "n"))
    assert _tree(ir.parse("(seq dummy (dummy))")) == ("seq", ("dummy",), ("dummy",))
    # integers, negative ones included, are NUM; anything else bare is a VAR, also `P+M` and `1.5` (IrParser.py:38-40, :50-51)
    assert _tree(ir.parse("(const_tile P+M -16)")) == ("const_tile", "P+M", -16)
    assert _tree(ir.parse("(/ x 1.5)")) == ("/", "x", "1.5")
    # a whole statement: store of two outputs from a load of two inputs
    got = _tree(ir.parse("(sloop 0 P+M 16 p (store (output A, B) (x (load (input X,Y) (index (tile p) fulltile)) 2) (index (elem h) (tile p))))"))
    assert got == ("sloop", 0, "P+M", 16, "p",
                   ("store", ("output", "A", "B"),
                    ("x", ("load", ("input", "X", "Y"), ("index", ("tile", "p"), ("fulltile",))), 2),
                    ("index", ("elem", "h"), ("tile", "p"))))


@pytest.mark.parametrize("name", UNSUPPORTED)
def test_other_programs_are_reported_unsupported(name):
    m = ir.recognise(UNSUPPORTED[name])
    assert not m and m.variant is None and m.reason


def test_grammar_details_of_the_reference_parser():
    t = ir.parse("(store (output A, B) (load (input X,Y) (index (tile m) fulltile)) (index (tile m) (elem -3))) ; trailing comment")
    assert t.op == "store" and t.args[0] == ir.Node("output", ("A", "B"))
    assert t.args[1].args[0].args == ("X", "Y")
    assert t.args[1].args[1].args[1] == ir.Node("fulltile") and t.args[2].args[1].args == (-3,)
    assert ir.parse("(index (fulltile) fulltile)").args[0] == ir.Node("fulltile")            # both spellings
    assert ir.parse("(sloop 0 P+M 16 p dummy)").args == (0, "P+M", 16, "p", ir.Node("dummy"))
    assert ir.parse(str(t)) == t                                                             # printing round-trips
    for bad, msg in (("(frobnicate 1 2)", "Unknown operation: frobnicate"), ("(+ 1 2", "Missing closing parenthesis"),
                     ("", "Unexpected end of input"), ("(", "Unexpected end of input"), ("(load (input X))", "load expects 2")):
        with pytest.raises(ValueError, match=msg.replace("(", r"\(").replace("+", r"\+")):
            ir.parse(bad)
    assert not ir.recognise("(+ 1 2") and "cannot parse" in ir.recognise("(+ 1 2").reason


def test_dataflow_summary_follows_accumulations_and_appends():
    df = ir.analyse(ir.parse(CANDIDATES["vanilla"][0]))
    assert df.inputs == {"X", "WQ", "WK", "WV", "K_cache", "V_cache"}
    assert df.stored["K_cache"].srcs == {"X", "WK"} and df.stored["K_cache"].ops == {"matmul"}
    assert df.stored["O2"].srcs == {"X", "WQ", "WK", "WV", "K_cache", "V_cache"}
    assert {"exp", "div", "rsum", "add", "matmul"} <= df.stored["O2"].ops and not df.squares
    assert df.stored["C_sum"].ops >= {"exp", "rsum", "add"}


def test_ir_file_reader(tmp_path):
    p = tmp_path / "cands.txt"
    p.write_text("\n".join(["# header", "0: " + CANDIDATES["vanilla"][0].replace("\n", " "), "",
                            "1: (seq dummydata)", "x7: (seq dummy)", "12:   " + UNSUPPORTED["unknown inputs"], "no colon here"]))
    got = ir.read_ir_file(str(p))
    assert [i for i, _ in got] == [0, 12]
    assert ir.recognise(got[0][1]).variant == "vanilla" and not ir.recognise(got[1][1])


def ir_file(tmp_path):
    lines = [f"{i}: " + c for i, c in enumerate([CANDIDATES["vanilla"][0], CANDIDATES["roco"][0], UNSUPPORTED["unknown inputs"],
                                                  CANDIDATES["keyformer"][1], CANDIDATES["qknorm"][0]])]
    p = tmp_path / "cands.txt"
    p.write_text("\n".join(lines))
    return str(p)


def test_candidates_of_a_file_are_selected_like_the_reference_flags(tmp_path):
    from triton_amd import benchmark
    path = ir_file(tmp_path)
    assert [(i, v) for i, _, v, *_ in benchmark.candidates_from_ir(path, 0, None)] == \
        [(0, "vanilla"), (1, "roco"), (2, None), (3, "keyformer"), (4, "qknorm")]
    assert [i for i, *_ in benchmark.candidates_from_ir(path, 1, 2)] == [1, 2]
    assert [i for i, *_ in benchmark.candidates_from_ir(path, 3, 10)] == [3, 4]
    assert benchmark.candidates_from_ir(path, 3, 1)[0][4] == {"tau": 1.5}          # constants read off the candidate


def test_evaluate_checks_the_case_file_against_the_variant(tmp_path, capsys):
    from triton_amd import evaluate
    case = tmp_path / "roco_llama_case0.txt"
    case.write_text(CANDIDATES["roco"][0])
    assert evaluate.main(["--t", "roco", "--case", str(case)]) == 0
    assert evaluate.main(["--t", "vanilla", "--case", str(case)]) == 2
    assert "recognised as roco" in capsys.readouterr().out


@pytest.mark.gpu
def test_benchmark_cli_times_recognised_candidates_and_records_the_rest(tmp_path):
    import json
    import math
    from triton_amd import benchmark
    cfgs = tmp_path / "c.json"
    cfgs.write_text(json.dumps([{"M": 16, "N": 512, "D": 64, "H": 8, "P": 40}]))
    out = tmp_path / "o.json"
    assert benchmark.main(["--ir", ir_file(tmp_path), "--end", "--configs", str(cfgs), "--output", str(out),
                           "--runs", "5", "--warmup", "2", "--topk", "3"]) == 0
    data = json.loads(out.read_text())
    assert [d["ir_id"] for d in data] == [0, 1, 2, 3, 4]
    assert all(d["error"] is None and 0 < d["execution_time_ms"] < 10 for d in data if d["ir_id"] != 2)
    assert data[2]["error"].startswith("unsupported IR") and math.isinf(data[2]["execution_time_ms"])
    assert data[0]["ir_expression"].startswith("(seq (ploop")


@pytest.mark.gpu
@pytest.mark.parametrize("variant,index", [(v, i) for table in (CANDIDATES, LINEAR) for v, c in table.items() for i in range(len(c))])
def test_recognised_candidate_runs_and_matches_the_oracle(variant, index):
    """parse -> recognise -> module -> run, as the reference's drivers go from a candidate to a timed module
    (vanilla_llama_benchmark.py:141-221): the module a candidate is mapped to, built with the constants read off the
    candidate, computes what the oracle says that workload computes."""
    import torch
    from oracle import ref
    from triton_amd import modules
    m = ir.recognise((CANDIDATES.get(variant) or LINEAR[variant])[index])
    assert m.variant == variant, m.reason
    g = torch.Generator().manual_seed(100 + index)

    def close(got, want, atol, rtol=1e-2):
        err = (got.float().cpu() - want.float()).abs()
        assert (err <= atol + rtol * want.float().abs()).all(), f"max abs err {err.max():.4g}"

    if variant in LINEAR:
        mod = modules.get(variant, "linear", **m.kwargs)
        if variant == "lora":
            M, N, P, R = 16, 256, 128, 32
            cpu = dict(X=ref.randn_half((M, N), g, 0, 0.5), W=ref.randn_half((N, P), g, 0, 0.1), A=ref.randn_half((N, R), g, 0, 0.1),
                       B=ref.randn_half((R, P), g, 0, 0.1))
            want = ref.lora(cpu["X"], cpu["W"], cpu["A"], cpu["B"])
        else:
            M, K, N = 16, 256, 192
            cpu = dict(X=ref.randn_half((M, K), g, 0, 0.5), W1=ref.randn_half((K, N), g, 0, 0.1), W2=ref.randn_half((K, N), g, 0, 0.1))
            want = ref.gated_mlp(cpu["X"], cpu["W1"], cpu["W2"], m.kwargs["gate"])
        t = {k: v.cuda() for k, v in cpu.items()}
        t["O"] = torch.zeros(tuple(want.shape), dtype=torch.float16, device="cuda")
        mod.forward(*[t[p] for p in mod.TENSOR_PARAMS])
        torch.cuda.synchronize()
        close(t["O"], want, 2e-2)
        return
    M, N, D, P = 16, 512, 64, 40
    H = N // D
    rnd = lambda *sh: ref.reference_recipe(sh, g) * 20
    cpu = dict(X=rnd(M, N), WQ=rnd(N, N), WK=rnd(N, N), WV=rnd(N, N), K_cache=rnd(H, P + M, D), V_cache=rnd(H, P + M, D))
    if variant == "prenorm":       # |X_norm| is about 1 whatever X's amplitude: keep the unscaled scores moderate
        for w in ("WQ", "WK", "WV"):
            cpu[w] = cpu[w] * 0.1
    cpu = {k: v.half() for k, v in cpu.items()}
    cpu["noise"] = torch.randn(H, M, P + M, generator=g).half()
    mod = modules.get(variant, "decode", head_dim=D, **m.kwargs)
    t = {k: v.cuda() for k, v in cpu.items()}
    t["O2"] = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    for c in ("C_out", "C_out1", "C_out2"):
        t[c] = torch.zeros(H, P + M, device="cuda")
    mod.forward(*[t[p] for p in mod.TENSOR_PARAMS])
    torch.cuda.synchronize()
    args = (cpu["X"], cpu["WQ"], cpu["WK"], cpu["WV"], cpu["K_cache"], cpu["V_cache"])
    if variant in ("vanilla", "prenorm"):
        want = ref.decode_append_vanilla(*args, P, D, prenorm=variant == "prenorm")
    elif variant == "qknorm":
        want = ref.decode_append_qknorm(*args, P, D)
    elif variant == "keyformer":
        want, pw = ref.decode_append_keyformer(*args, cpu["noise"], P, D, tau=m.kwargs["tau"])
        close(t["C_out"], pw.sum(1), 1e-5, 5e-3)
    else:
        want, s1, s2 = ref.decode_append_roco(*args, P, D)
        close(t["C_out1"], s1, 1e-5, 5e-3); close(t["C_out2"], s2, 1e-6, 5e-3)
    close(t["O2"], ref.flatten_token_major(want), 2e-3 if variant != "prenorm" else 2e-2)


def test_printing_round_trips_on_random_trees():
    """parse(str(tree)) == tree for randomly generated well-formed programs (hypothesis)."""
    from hypothesis import given, settings, strategies as st
    names = st.sampled_from(["X", "WQ", "K_cache", "O2", "C_sum", "noise", "T1"])
    atoms = st.one_of(st.integers(-64, 4096), st.sampled_from(["m", "n", "p", "P+M", "N", "1.5"]))
    idx = st.lists(st.one_of(st.just(ir.Node("fulltile")), st.builds(lambda v: ir.Node("tile", (v,)), st.sampled_from(["m", "n", "p"])),
                             st.builds(lambda v: ir.Node("elem", (v,)), st.sampled_from(["h", "m"])),
                             st.builds(lambda a, b: ir.Node("const_tile", (a, b)), atoms, atoms)), min_size=1, max_size=3)
    index = st.builds(lambda xs: ir.Node("index", tuple(xs)), idx)
    named = st.builds(lambda k, ns: ir.Node(k, tuple(ns)), st.sampled_from(["input", "output", "tensor"]), st.lists(names, min_size=1, max_size=3, unique=True))
    load = st.builds(lambda t, i: ir.Node("load", (t, i)), named, index)
    value = st.recursive(st.one_of(load, atoms), lambda kids: st.one_of(
        st.builds(lambda op, a, b: ir.Node(op, (a, b)), st.sampled_from(["+", "-", "x", "/", "*"]), kids, kids),
        st.builds(lambda op, a: ir.Node(op, (a,)), st.sampled_from(["exp", "sqr", "sqrt", "sigmoid"]), kids),
        st.builds(lambda a, ax: ir.Node("rsum", (a, ax)), kids, st.integers(0, 2)),
        st.builds(lambda a, ax: ir.Node("bcast", (a, ax)), kids, st.integers(0, 3))), max_leaves=8)
    store = st.builds(lambda t, v, i: ir.Node("store", (t, v, i)), named, value, index)
    stmt = st.recursive(st.one_of(store, st.just(ir.Node("dummy"))), lambda kids: st.one_of(
        st.builds(lambda xs: ir.Node("seq", tuple(xs)), st.lists(kids, min_size=1, max_size=3)),
        st.builds(lambda k, a, b, t, v, body: ir.Node(k, (a, b, t, v, body)), st.sampled_from(["ploop", "sloop"]), atoms, atoms,
                  st.integers(1, 128), st.sampled_from(["m", "n", "p", "h"]), kids)), max_leaves=5)

    @settings(max_examples=150, deadline=None)
    @given(stmt)
    def check(tree):
        assert ir.parse(str(tree)) == tree
        ir.recognise(tree)                       # never raises: a Match either way
    check()
