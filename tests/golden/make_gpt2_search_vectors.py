"""Writes tests/golden/gpt2_search_vectors.npz: the per-step logits of the reference's own greedy and beam
search golden tests, so that the expected token sequences those tests hold pin ArgMax, BeamSearch_Cpu::SelectTop and
BeamSearchScorer::Process / Finalize without ONNX Runtime.

The golden tests are ModelTests.GreedySearchGptFp32 and ModelTests.BeamSearchGptFp32
(/root/reference/test/model_tests.cpp:57-130): prompts and expected outputs are the integer arrays written there, the
model is the data file test/models/hf-internal-testing/tiny-random-gpt2-fp32/past.onnx (5 layers, 4 heads of 8,
vocabulary 1000).  The reference's C++ cannot run here (it needs ONNX Runtime), so this script
  * decodes the ONNX protobuf by hand (wire format only; nothing in the file is executed),
  * evaluates the graph's six operator kinds in numpy fp32 (Cast, EmbedLayerNormalization, Attention,
    SkipLayerNormalization, FastGelu, MatMul; the com.microsoft operators follow their published contrib-op
    definitions), recomputing the whole sequence at every step instead of carrying a KV cache,
  * drives the oracle's search functions with those logits, and
  * REFUSES to write anything unless the resulting sequences equal the reference's expected outputs.
What is stored: prompts, expected outputs, search options, and for every step along the golden trajectory the logits
and (beam search) the token rows they were computed for -- inputs and expected outputs only.
tests/test_gpt2_golden.py replays them through the oracle (CPU) and through the HIP kernels (GPU); each replay also
checks that the sequences it feeds back are the ones the logits were computed for.

Run where /root/reference exists:  python tests/golden/make_gpt2_search_vectors.py"""
import os
import struct
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import orc_lib  # noqa: E402

MODEL = "/root/reference/test/models/hf-internal-testing/tiny-random-gpt2-fp32/past.onnx"
PAD = EOS = 98  # genai_config.json beside the model

# test/model_tests.cpp:58-63
GREEDY_PROMPT = np.array([[0, 0, 0, 52], [0, 0, 195, 731]], np.int32)
GREEDY_EXPECTED = np.array([[0, 0, 0, 52, 204, 204, 204, 204, 204, 204],
                            [0, 0, 195, 731, 731, 114, 114, 114, 114, 114]], np.int32)
# test/model_tests.cpp:93-102; num_beams 4, length_penalty 1.0, max_length 20 (:112-118)
BEAM_PROMPT = np.array([[0, 0, 0, 0, 0, 52, 195, 731, 321, 301, 734, 620],
                        [41, 554, 74, 622, 206, 222, 75, 223, 221, 198, 224, 572],
                        [0, 0, 0, 52, 328, 219, 328, 206, 288, 227, 896, 328]], np.int32)
BEAM_EXPECTED = np.array([
    [0, 0, 0, 0, 0, 52, 195, 731, 321, 301, 734, 620, 131, 131, 131, 181, 638, 638, 638, 638],
    [41, 554, 74, 622, 206, 222, 75, 223, 221, 198, 224, 572, 292, 292, 292, 292, 292, 292, 292, 292],
    [0, 0, 0, 52, 328, 219, 328, 206, 288, 227, 896, 328, 328, 669, 669, 669, 669, 669, 669, 669]], np.int32)


# ---- protobuf wire format ------------------------------------------------------------------------------------
def _varint(b, i):
    r = s = 0
    while True:
        c = b[i]
        i += 1
        r |= (c & 0x7F) << s
        s += 7
        if c < 0x80:
            return r, i


def _fields(b):
    i, n = 0, len(b)
    while i < n:
        key, i = _varint(b, i)
        f, w = key >> 3, key & 7
        if w == 0:
            v, i = _varint(b, i)
        elif w == 1:
            v, i = b[i:i + 8], i + 8
        elif w == 2:
            ln, i = _varint(b, i)
            v, i = b[i:i + ln], i + ln
        elif w == 5:
            v, i = b[i:i + 4], i + 4
        else:
            raise ValueError("wire type %d" % w)
        yield f, w, v


def _tensor(b):  # TensorProto: dims 1, data_type 2, name 8, raw_data 9
    dims, dt, name, raw = [], None, None, None
    for f, w, v in _fields(b):
        if f == 1:
            if w == 0:
                dims.append(v)
            else:
                j = 0
                while j < len(v):
                    x, j = _varint(v, j)
                    dims.append(x)
        elif f == 2:
            dt = v
        elif f == 8:
            name = bytes(v).decode()
        elif f == 9:
            raw = bytes(v)
    assert dt == 1 and raw is not None, (name, dt)  # every initializer of this model is fp32 raw data
    return name, np.frombuffer(raw, np.float32).reshape(dims).copy()


def _node(b):  # NodeProto: input 1, output 2, op_type 4, attribute 5 (AttributeProto: name 1, f 2, i 3)
    d = {"in": [], "out": [], "attr": {}}
    for f, w, v in _fields(b):
        if f == 1:
            d["in"].append(bytes(v).decode())
        elif f == 2:
            d["out"].append(bytes(v).decode())
        elif f == 4:
            d["op"] = bytes(v).decode()
        elif f == 5:
            name = val = None
            for f2, w2, v2 in _fields(v):
                if f2 == 1:
                    name = bytes(v2).decode()
                elif f2 == 2:
                    val = struct.unpack("<f", v2)[0]
                elif f2 == 3:
                    val = v2
            d["attr"][name] = val
    return d


def load_graph(path):
    b = memoryview(open(path, "rb").read())
    nodes, weights = [], {}
    for f, w, v in _fields(b):
        if f == 7:  # ModelProto.graph
            for f2, w2, v2 in _fields(v):
                if f2 == 1:
                    nodes.append(_node(v2))
                elif f2 == 5:
                    name, arr = _tensor(v2)
                    weights[name] = arr
    return nodes, weights


# ---- the graph's operators in numpy fp32 ----------------------------------------------------------------------
F = np.float32


def layer_norm(x, gamma, beta, eps):
    mean = x.mean(-1, keepdims=True, dtype=F)
    d = x - mean
    var = (d * d).mean(-1, keepdims=True, dtype=F)
    return (d / np.sqrt(var + F(eps))) * gamma + beta


def attention(x, w, bias, heads):
    """com.microsoft.Attention, unidirectional, empty past, all-ones mask: x [B,S,H] -> [B,S,H]."""
    B, S, H = x.shape
    qkv = x @ w + bias
    q, k, v = (qkv[..., i * H:(i + 1) * H].reshape(B, S, heads, H // heads).transpose(0, 2, 1, 3) for i in range(3))
    s = (q @ k.transpose(0, 1, 3, 2)) * F(1.0 / np.sqrt(H // heads))
    s = np.where(np.tril(np.ones((S, S), bool)), s, F(-3.4028234663852886e+38))
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s)
    p = e / e.sum(-1, keepdims=True, dtype=F)
    return (p @ v).transpose(0, 2, 1, 3).reshape(B, S, H)


def fast_gelu(x, bias):
    x = x + bias
    return x * (F(0.5) + F(0.5) * np.tanh(x * (F(0.035677408136300125) * x * x + F(0.7978845608028654))))


def run_graph(nodes, weights, ids):
    """Logits [rows, vocab] of the last position for token rows `ids` [rows, S] (positions 0..S-1, no padding:
    the prompts' zeros are ordinary tokens, the pad id is 98)."""
    B, S = ids.shape
    env = dict(weights)
    env["input_ids"] = ids.astype(np.int64)
    env["position_ids"] = np.broadcast_to(np.arange(S, dtype=np.int64), (B, S))
    env["attention_mask"] = np.ones((B, S), np.int32)
    for n in nodes:
        i = [env.get(x) if x else None for x in n["in"]]
        op = n["op"]
        if op == "Cast":
            out = [i[0].astype(np.int32)]
        elif op == "EmbedLayerNormalization":
            emb = i[2][i[0]] + i[3][i[8]]
            out = [layer_norm(emb, i[5], i[6], n["attr"]["epsilon"]), None, emb]
        elif op == "Attention":
            assert n["attr"]["unidirectional"] == 1
            out = [attention(i[0], i[1], i[2], n["attr"]["num_heads"]), None]
        elif op == "MatMul":
            out = [i[0] @ i[1]]
        elif op == "SkipLayerNormalization":
            s = i[0] + i[1] + i[4]
            out = [layer_norm(s, i[2], i[3], n["attr"]["epsilon"]), None, None, s]
        elif op == "FastGelu":
            out = [fast_gelu(i[0], i[1])]
        else:
            raise ValueError(op)
        for name, val in zip(n["out"], out):
            if name and val is not None:
                assert val.dtype in (np.float32, np.int32), (op, val.dtype)
                env[name] = val
    return np.ascontiguousarray(env["logits"][:, -1, :])


# ---- the two golden generations -----------------------------------------------------------------------------
def greedy(orc, nodes, weights):
    """GreedySearch_Cpu::SelectTop + AppendNextTokensToSequences (src/search.cpp:178-201,256-296)."""
    seq = GREEDY_PROMPT.copy()
    max_length = GREEDY_EXPECTED.shape[1]
    eos_seen = np.zeros(len(seq), bool)
    steps = []
    while seq.shape[1] < max_length and not eos_seen.all():
        logits = run_graph(nodes, weights, seq)
        steps.append(logits)
        tok = orc.argmax_batch(logits)
        tok = np.where(eos_seen, PAD, tok).astype(np.int32)
        eos_seen |= tok == EOS
        seq = np.concatenate([seq, tok[:, None]], 1)
    return seq, np.stack(steps)


def beam(orc, nodes, weights, beams=4, length_penalty=1.0, early_stopping=True):
    """BeamSearch_Cpu::SelectTop (src/search.cpp:101-176) until the scorer is done or max_length is reached, then
    Finalize and hypothesis 0 of every batch entry (src/search.cpp:383-395)."""
    batch, plen = BEAM_PROMPT.shape
    max_length = BEAM_EXPECTED.shape[1]
    ref = orc_lib.BeamScorer(orc, batch, beams, max_length, PAD, [EOS], length_penalty, early_stopping)
    seq = np.zeros((batch * beams, max_length), np.int32)
    seq[:, :plen] = np.repeat(BEAM_PROMPT, beams, axis=0)
    length = plen
    steps, inputs = [], []
    while length < max_length and not ref.is_done():
        logits = run_graph(nodes, weights, seq[:, :length])
        steps.append(logits)
        inputs.append(seq.copy())
        sc, tok, idx, _ = orc.beam_select_top(logits, batch, beams, ref.next_scores)
        ref.process(seq, length, sc, tok, idx)
        nxt = np.zeros_like(seq)
        orc.lib.orc_beam_append(seq.reshape(-1), nxt.reshape(-1), batch * beams, max_length, length,
                                ref.next_indices, ref.next_tokens)
        seq, length = nxt, length + 1
    ref.finalize(seq, length)
    out = np.stack([np.pad(ref.hyp(b, 0)[0], (0, max_length))[:max_length] for b in range(batch)])
    return out, np.stack(steps), np.stack(inputs)


def main():
    nodes, weights = load_graph(MODEL)
    orc = orc_lib.Oracle()
    g_seq, g_logits = greedy(orc, nodes, weights)
    assert np.array_equal(g_seq, GREEDY_EXPECTED), g_seq
    b_seq, b_logits, b_inputs = beam(orc, nodes, weights)
    assert np.array_equal(b_seq, BEAM_EXPECTED), b_seq
    path = os.path.join(HERE, "gpt2_search_vectors.npz")
    np.savez_compressed(path, greedy_prompt=GREEDY_PROMPT, greedy_expected=GREEDY_EXPECTED, greedy_logits=g_logits,
                        beam_prompt=BEAM_PROMPT, beam_expected=BEAM_EXPECTED, beam_logits=b_logits, beam_inputs=b_inputs,
                        options=np.array([PAD, EOS, 4], np.int32))
    print("wrote", path, g_logits.shape, b_logits.shape, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
