"""GPU parity of the device sampler (ptm_sample_token, ptm_decode_sample) against the CPU oracle's restatement of
GGUFModel::sample_token (torch/io/gguf_model.h:7658-7751) and of the repetition penalty (:4926-4938).

Bar: the same token as the oracle for the same uniform draw r whenever r is further than GAP_TOL from the edges of
that token's interval of the cumulative distribution (device expf and glibc expf may differ in the last bit, which
moves the edges by ~1e-7)."""
import numpy as np
import pytest
import torch

from prometorch_amd import ops
from prometorch_amd.testing import synth
from prometorch_amd._lib import PtmError

pytestmark = pytest.mark.gpu

GAP_TOL = 1e-5



def gap_tol(vocab, temperature, top_k):
    """Over the whole vocabulary (top-k off) the reference's softmax denominator and running sums are sequential fp32 sums of
    up to 151 936 terms, which drift from the exact sums by a few 1e-4 relative at that length (measured: the reference's
    probabilities then add up to 1 +- 3e-4 in float64); the device sums there are order-independent fixed-point ones.  A draw
    closer than this to an interval edge of the reference's CDF may land on a neighbouring token."""
    return max(GAP_TOL, 3e-9 * vocab) if wide(vocab, temperature, top_k) else GAP_TOL


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def gpu_sample(x, temperature, top_k, top_p, r, counts=None, penalty=1.0):
    ws = torch.empty(ops.sampler_workspace_bytes(), dtype=torch.uint8, device="cuda")
    ws.fill_(0xAB)  # contents must not matter
    out = torch.full((1,), -7, dtype=torch.int64, device="cuda")
    ops.sample_token(cu(x), x.size, None if counts is None else cu(counts.astype(np.int32)), temperature, top_k, top_p,
                     penalty, cu(np.array([r], np.float32)), ws, out)
    torch.cuda.synchronize()
    return int(out.item())


def check_wide_draw(tok_g, tok_o, gap, probs, r, tol, vocab):
    """The bar of the whole-vocabulary path: the reference's token when the draw is clear of its interval's edges, otherwise a
    kept token whose interval of the reference's CDF (fp32, index order: the sum the reference walks) holds the draw to within
    tol.  Where the reference's running sum stops short of the draw its loop returns the last id; the device's sum may reach
    the draw there, and the other way round."""
    cdf = np.cumsum(probs)
    fell_off = cdf[-1] < r
    if (gap > tol and not fell_off) or r == 0.0:
        assert tok_g == tok_o, (float(r), gap)
        return
    assert (tok_g == vocab - 1 and r > cdf[-1] - tol) or \
        (probs[tok_g] > 0 and cdf[tok_g] + tol >= r and (tok_g == 0 or cdf[tok_g - 1] - tol <= r)), (float(r), tok_g, tok_o)


def wide(vocab, temperature, top_k):
    """top-k off or beyond the candidate list: the sampler's passes over the whole vocabulary"""
    return temperature >= 1e-6 and not (1 <= top_k <= 1024 and top_k < vocab)


def test_mt19937_uniforms_are_the_reference_sequence(po):
    g = po.MT19937(42)
    want = [g.uniform01() for _ in range(300)]
    assert ops.mt19937_uniforms(42, 0, 300) == want
    assert ops.mt19937_uniforms(42, 100, 50) == want[100:150]
    assert abs(want[0] - 0.3745401) < 1e-7


def test_sample_token_cases_vs_oracle_and_reference_golden(dev, po, golden_sampling):
    rng = po.MT19937(42)
    checked = 0
    for i, (vocab, kind, temperature, top_k, top_p) in enumerate(synth.SAMPLING_CASES):
        x = synth.sampling_logits(i)
        r = rng.uniform01() if temperature >= 1e-6 else 0.0
        tok_o, gap = po.sample_token(x, temperature, top_k, top_p, r)
        assert tok_o == int(golden_sampling[i])        # the oracle is the compiled reference here
        tok_g = gpu_sample(x, temperature, top_k, top_p, r)
        print(i, vocab, kind, temperature, top_k, top_p, "r %.6f gap %.2e" % (r, gap), tok_g, tok_o, flush=True)
        if gap > gap_tol(vocab, temperature, top_k):
            assert tok_g == tok_o, (i, wide(vocab, temperature, top_k))
            checked += 1
    assert checked >= 36


@pytest.mark.parametrize("vocab,kind_case,temperature,top_k,top_p", [(1000, 0, 0.8, 40, 0.9), (151936, 12, 0.8, 40, 0.9),
                                                                      (151936, 18, 1.0, 1024, 0.95), (1000, 3, 1.3, 7, 1.0),
                                                                      (151936, 19, 0.5, 2, 0.5),
                                                                      # the wide path: top-k off, top-k beyond the list
                                                                      (1000, 1, 1.0, 0, 1.0), (1000, 6, 0.8, 0, 0.9),
                                                                      (1000, 9, 0.8, 1000, 0.95), (151936, 18, 0.6, 0, 0.9),
                                                                      (151936, 12, 0.8, 5000, 0.9), (151936, 16, 1.0, 0, 1.0),
                                                                      (151936, 12, 2.5, 0, 0.5), (1000, 3, 1.0, 0, 0.7)])
def test_sample_token_many_draws(dev, po, vocab, kind_case, temperature, top_k, top_p):
    """The whole inverse CDF: 64 draws spread over (0, 1) plus the edges."""
    x = synth.sampling_logits(kind_case)
    assert x.size == vocab
    rs = list(np.random.default_rng(kind_case).random(60).astype(np.float32)) + [0.0, 1e-30, 0.99999994, 0.5]
    checked = 0
    for r in rs:
        tok_o, gap, probs = po.sample_token(x, temperature, top_k, top_p, float(r), want_probs=True)
        tok_g = gpu_sample(x, temperature, top_k, top_p, float(r))
        if wide(vocab, temperature, top_k):
            # a flat distribution over 151 936 tokens has intervals narrower than the drift of the reference's own running sum
            check_wide_draw(tok_g, tok_o, gap, probs, r, gap_tol(vocab, temperature, top_k), vocab)
            checked += 1
        elif gap > GAP_TOL or r == 0.0:
            assert tok_g == tok_o, (float(r), gap)
            checked += 1
    assert checked >= 55


def test_sample_token_with_repetition_penalty(dev, po):
    vocab = 5000
    g = synth.rng_for(81)
    x = (3 * g.standard_normal(vocab, dtype=np.float32)).astype(np.float32)
    top = np.argsort(x)[::-1]
    generated = [int(top[0])] * 3 + [int(top[1]), int(top[5]), int(top[5]), int(np.argmin(x)), 17, 17, 17, 17]
    counts = np.bincount(generated, minlength=vocab)
    for penalty in (1.1, 1.5, 1.0):
        xp = po.repetition_penalty(x, generated, penalty)
        for r in (0.05, 0.31, 0.77, 0.93):
            tok_o, gap = po.sample_token(xp, 0.8, 40, 0.9, r)
            tok_g = gpu_sample(x, 0.8, 40, 0.9, r, counts=counts, penalty=penalty)
            if gap > GAP_TOL:
                assert tok_g == tok_o, (penalty, r)
        # greedy over the penalised logits
        assert gpu_sample(x, 0.0, 40, 0.9, 0.5, counts=counts, penalty=penalty) == int(np.argmax(xp))
    # penalty 1.5 three times on the best token must dethrone it
    assert int(np.argmax(po.repetition_penalty(x, generated, 1.5))) != int(top[0])


def test_sample_token_greedy_ties_and_edges(dev, po):
    x = np.zeros(3000, np.float32)
    x[[5, 77, 2999]] = 4.0
    assert gpu_sample(x, 0.0, 1, 1.0, 0.9) == 5                       # argmax: lowest index of the tied maxima
    assert gpu_sample(x, 1.0, 2, 1.0, 0.99) == 2999                   # top-2 keeps all three ties; last interval
    assert gpu_sample(x, 1.0, 2, 1.0, 0.5) == 77
    assert gpu_sample(x, 1.0, 3, 1.0, 0.0) == 0                       # r = 0: index 0, whatever its probability
    x = np.array([-0.0, 0.0, -1.0, 0.0], np.float32)                  # -0 and +0 are the same value to the reference
    tok_o, _ = po.sample_token(x, 1.0, 2, 1.0, 0.5)
    assert gpu_sample(x, 1.0, 2, 1.0, 0.5) == tok_o
    flat = np.zeros(5000, np.float32)                                 # 5000 logits tie at the threshold: more than the list holds
    tok_o, _ = po.sample_token(flat, 1.0, 4, 1.0, 0.5)                # the reference keeps every tie: uniform over all 5000
    assert gpu_sample(flat, 1.0, 4, 1.0, 0.5) == tok_o
    assert gpu_sample(flat, 0.0, 1, 1.0, 0.5) == 0                    # greedy over 5000 equal maxima: the lowest index
    flat2 = np.zeros(2048, np.float32)                                # exactly as many as it holds
    tok_o, _ = po.sample_token(flat2, 1.0, 4, 1.0, 0.5)
    assert gpu_sample(flat2, 1.0, 4, 1.0, 0.5) == tok_o


@pytest.mark.parametrize("top_k,top_p", [(40, 1.0), (40, 0.9), (300, 0.5), (1, 1.0)])
def test_more_ties_at_the_threshold_than_the_candidate_list_holds(dev, po, top_k, top_p):
    """A plateau of 3000 equal logits at the top-k cut (above it a few larger ones, below it the rest): the reference keeps every
    tie (gguf_model.h:7682-7691), so more than 2048 candidates survive and the draw comes from the overflow kernel, which walks
    the whole vocabulary; the bar is the wide path's (order-independent sums)."""
    rng = np.random.default_rng(91)
    vocab = 20000
    x = (rng.standard_normal(vocab) * 0.5 - 3.0).astype(np.float32)
    plateau = rng.choice(vocab, 3000, replace=False)
    x[plateau] = 1.25
    x[plateau[:7]] = np.array([3.0, 2.5, 2.5, 2.0, 1.75, 1.5, 1.5], np.float32)   # 7 above the plateau: k = 40 cuts inside it
    tol = max(GAP_TOL, 3e-9 * vocab)
    checked = 0
    for r in list(rng.random(24).astype(np.float32)) + [0.0, 0.99999994]:
        tok_o, gap, probs = po.sample_token(x, 0.9, top_k, top_p, float(r), want_probs=True)
        tok_g = gpu_sample(x, 0.9, top_k, top_p, float(r))
        if top_k == 1:
            assert tok_g == tok_o          # one maximum, no tie at k = 1: the narrow path
            continue
        check_wide_draw(tok_g, tok_o, gap, probs, r, tol, vocab)
        checked += 1
    assert top_k == 1 or checked >= 20


def test_sample_token_argument_errors(dev):
    x = np.zeros(100, np.float32)
    for temperature, top_k, top_p in ((0.8, 40, 0.0), (0.8, 0, -1.0)):
        with pytest.raises(PtmError):
            gpu_sample(x, temperature, top_k, top_p, 0.5)


def build_tiny(seeds):
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    return cfg, layers, head


@pytest.mark.parametrize("use_graph", [True, False])
@pytest.mark.parametrize("temperature,top_k,top_p,penalty", [(0.8, 40, 0.9, 1.1), (1.2, 8, 1.0, 1.0), (0.0, 40, 0.9, 1.3),
                                                             (0.9, 0, 0.92, 1.05), (1.1, 0, 1.0, 1.0)])  # top-k off
def test_decoder_sampled_generation_vs_oracle_loop(dev, po, seeds, use_graph, temperature, top_k, top_p, penalty):
    """The reference's decode loop (api_handlers.h:848-923): penalise with the generated tokens, sample, feed back."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    om = po.OracleModel(cfg, layers, head, 96, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=use_graph)
    prompt = [int(t) for t in synth.rng_for(82).integers(0, cfg["vocab"], 9)]
    for t in prompt[:-1]:
        om.step(t)
        dec.step(t)
    n = 40
    us = ops.mt19937_uniforms(42, 0, n)
    dec.sampling_begin(temperature, top_k, top_p, penalty)
    got = dec.sample(prompt[-1], us[:25]) 
    got += dec.sample(got[-1], us[25:])            # a second run continues the same generation (counts are kept)
    tok, generated, min_gap = prompt[-1], [], 1.0
    for st in range(n):
        om.step(tok)
        lg = po.repetition_penalty(om.logits, generated, penalty) if generated else om.logits
        tok, gap = po.sample_token(lg, temperature, top_k, top_p, us[st])
        if gap <= 1e-4:
            break                                  # a draw on an interval edge: both answers are legitimate, stop comparing
        min_gap = min(min_gap, gap)
        assert got[st] == tok, (st, gap)
        generated.append(tok)
    print("compared %d sampled steps, smallest gap %.2e" % (len(generated), min_gap), flush=True)
    assert len(generated) >= 20
    # sampling_begin forgets the history: the same draws from the same state reproduce the same tokens
    dec.set_past_len(len(prompt) - 1)
    dec.sampling_begin(temperature, top_k, top_p, penalty)
    assert dec.sample(prompt[-1], us) == got
    dec.close()


def test_one_decoder_serves_requests_of_every_parameter_class(dev, po, seeds):
    """A serving loop calls sampling_begin per request on ONE decoder.  The sampler's launch sequence depends on the parameters
    (candidate list; whole-vocabulary passes with / without the top-k select and the nucleus walk), and the sampled step is a
    captured graph: a request of another class must not replay the previous class's graph.  Each request is checked against
    the oracle's penalise -> sample -> feed-back loop (api_handlers.h:848-923, gguf_model.h:7658-7751)."""
    from prometorch_amd.decode import Decoder
    cfg = dict(synth.TINY, vocab=2048)   # room for a top-k beyond the candidate list (1024) that is still below the vocabulary
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    dec = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=True)
    prompt = [int(t) for t in synth.rng_for(85).integers(0, cfg["vocab"], 7)]
    for t in prompt[:-1]:
        dec.step(t)
    n = 24
    requests = [(0.8, 40, 0.9, 1.1),      # candidate list
                (0.8, 0, 0.9, 1.0),       # top-k off, nucleus walk
                (0.8, 1500, 1.0, 1.05),   # top-k beyond the list, no nucleus
                (0.9, 1500, 0.85, 1.0),   # both
                (1.1, 0, 1.0, 1.0),       # neither
                (0.0, 40, 0.9, 1.2),      # greedy
                (0.8, 40, 0.9, 1.1),      # the first class again
                (0.7, 64, 0.95, 1.0)]     # same class, other values: served by the same graph through the device copy
    compared = []
    for req, (temperature, top_k, top_p, penalty) in enumerate(requests):
        us = ops.mt19937_uniforms(42, 100 * req, n)
        dec.set_past_len(len(prompt) - 1)
        dec.sampling_begin(temperature, top_k, top_p, penalty)
        got = dec.sample(prompt[-1], us[:9]) 
        got += dec.sample(got[-1], us[9:])
        assert dec.L.ptm_decode_graph_state(dec.h, 1) == 1, req
        om = po.OracleModel(cfg, layers, head, 96, kv_fp16=True)
        for t in prompt[:-1]:
            om.step(t)
        tol = gap_tol(cfg["vocab"], temperature, top_k) * 10
        tok, generated = prompt[-1], []
        for st in range(n):
            om.step(tok)
            lg = po.repetition_penalty(om.logits, generated, penalty) if generated else om.logits
            tok, gap = po.sample_token(lg, temperature, top_k, top_p, us[st])
            if gap <= max(tol, 1e-4):
                break                                  # a draw on an interval edge: both answers are legitimate
            assert got[st] == tok, (req, st, gap)
            generated.append(tok)
        compared.append(len(generated))
    print("sampled steps compared per request:", compared, flush=True)
    assert min(compared) >= 8 and sum(compared) >= 0.6 * n * len(requests), compared
    dec.close()


def test_decoder_sampling_errors(dev, seeds):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    dec = Decoder(cfg, layers, head, max_seq=32, kv_fp16=True, use_graph=False)
    with pytest.raises(PtmError):
        dec.sample(1, [0.5])                       # no sampling_begin yet
    with pytest.raises(PtmError):
        dec.sampling_begin(0.8, 40, 0.0)           # top-p must be positive
    dec.sampling_begin(0.8, 40, 0.9)
    with pytest.raises(PtmError):
        dec.sample(1, [0.5] * 33)                  # would overflow the cache
    assert len(dec.sample(1, [0.5] * 4)) == 4
    dec.close()


def test_generate_loop_with_stop_tokens(dev, po, seeds):
    """ptm_decode_generate against the reference's loop restated with the oracle: sample, stop on a stop id (not
    emitted), feed back; and the decoder's position afterwards counts exactly the tokens that were fed."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    params = (0.9, 30, 0.95, 1.2)
    us = ops.mt19937_uniforms(42, 0, 50)

    def oracle_loop(prompt, stops, min_gap=1e-4):
        om = po.OracleModel(cfg, layers, head, 96, kv_fp16=True)
        for t in prompt[:-1]:
            om.step(t)
        tok, gen, clear = prompt[-1], [], 0
        for st in range(len(us)):
            om.step(tok)
            lg = po.repetition_penalty(om.logits, gen, params[3]) if gen else om.logits
            tok, gap = po.sample_token(lg, params[0], params[1], params[2], us[st])
            if gap > min_gap and clear == st:
                clear = st + 1          # draws so far all sit clear of their interval edges
            if tok in stops:
                break
            gen.append(tok)
        return gen, om, clear

    # a one-token prompt: no prefill, the decode path alone, which follows the oracle to ~1e-6 -- the loop logic exactly
    prompt = [int(synth.rng_for(83).integers(0, cfg["vocab"]))]
    free_run, _, clear = oracle_loop(prompt, ())
    assert clear == len(us), "a draw sits on an interval edge: pick other draws"
    dec = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=True)
    assert dec.generate(prompt, us, *params) == free_run
    for cut in (0, 5, 15, 16, 17, 33, 49):  # a stop at the first token, inside a run of 16, on its edges, at the very end
        stop = free_run[cut]
        first = free_run.index(stop)
        want, om, _ = oracle_loop(prompt, (stop, cfg["vocab"] + 5))
        assert want == free_run[:first]
        dec.set_past_len(0)
        got = dec.generate(prompt, us, *params, stop_ids=(stop, cfg["vocab"] + 5))
        assert got == want, cut
        # position: the prompt and every generated token were fed; one more step must see exactly that context
        probe = 11
        t_o = om.step(probe)
        t_g = dec.step(probe)
        assert t_g == t_o and np.abs(dec.logits() - om.logits).max() / om.logits.std() <= 1e-3, cut
    # a longer prompt goes through the prefill GEMMs (fp16 operands): the streams agree while the draws stay clear of
    # the interval edges by more than that noise
    prompt = [int(t) for t in synth.rng_for(84).integers(0, cfg["vocab"], 9)]
    want, _, clear = oracle_loop(prompt, (), min_gap=3e-2)
    dec.set_past_len(0)
    got = dec.generate(prompt, us, *params)
    assert len(got) == len(us) and got[:clear] == want[:clear] and clear >= 3
    dec.set_past_len(0)
    with pytest.raises(PtmError):
        dec.generate(prompt, [0.5] * 200, *params)          # does not fit the cache
    dec.close()
