"""The greedy decode driver over the KV-cached terms.

The reference's driver (catgrad-llm/examples/llama/main.rs:114-169) runs the whole sequence again for
every token, reads the sampled token with to_vec and pushes it onto the prompt.  `CachedRunner` is the
same loop over the KV-cached terms of this package (llama.LlamaPrefill / LlamaDecode and the
Qwen-MoE-layout ones): a prefill once, then one token per run, the cache tensors handed to the
evaluator by value so that a step may append to them in place.
"""
import numpy as np

from .. import abi
from ..interpreter import Interpreter, Parameters, stdlib
from . import llama


def interpreter(be, arrays):
    """An Interpreter whose Parameters hold `arrays` (path -> numpy array, or a ready Parameters)."""
    if isinstance(arrays, Parameters):
        return Interpreter(be, stdlib(), arrays)
    P = Parameters()
    for k, a in arrays.items():
        P[k] = be.tensor(a)
    return Interpreter(be, stdlib(), P)


class CachedRunner:
    """Greedy decoding with the KV-cached terms (prefill once, then one token per run)."""

    def __init__(self, be, cfg, arrays, max_positions, prefill_cls=None, decode_cls=None):
        """prefill_cls / decode_cls: the KV-cached term classes (default Llama's; the Qwen-MoE-layout
        ones take ids of shape [B, S])."""
        self.be, self.cfg = be, cfg
        self.prefill_cls = prefill_cls or llama.LlamaPrefill
        self.it = interpreter(be, arrays)
        self.cos, self.sin = self.it.run(llama.RopeTables(cfg).term(), [max_positions])
        self.decode_term = (decode_cls or llama.LlamaDecode)(cfg).term()
        self.kv = None
        self.pos = 0
        self._prefill_terms = {}

    def prefill(self, ids):
        ids = np.asarray(ids, np.uint32)
        ids = ids.reshape(1, -1) if ids.ndim == 1 else ids
        n = ids.shape[1]
        self.batch = ids.shape[0]
        if n not in self._prefill_terms:      # the term depends on the prompt length only
            self._prefill_terms[n] = self.prefill_cls(self.cfg, n).term()
        term = self._prefill_terms[n]
        out = self.it.run(term, [self.be.tensor(ids), self.cos, self.sin])
        self.kv = out[2:]
        self.pos = ids.shape[1]
        return out[0], out[1]

    def step(self, token):
        """`token`: an int (or one per batch row), or the token tensor of the previous step (stays on
        the device)."""
        if isinstance(token, abi.Tensor):
            ids = self.be.reshape(token, [self.batch, 1])
        else:
            ids = self.be.tensor(np.asarray(token, np.uint32).reshape(self.batch, 1))
        # the cache tensors are given away (Interpreter::run takes its values by value): the step may
        # then append to them in place
        out = self.it.run(self.decode_term, [ids, self.pos, self.cos, self.sin] + self.kv,
                          moved=range(4, 4 + len(self.kv)))
        self.kv = out[2:]
        self.pos += 1
        return out[0], out[1]

    def _host_tokens(self, tok):
        """The sampled token of every batch row: an int for one row, a list of ints for several."""
        t = self.be.to_vec(tok).reshape(-1)
        return int(t[0]) if self.batch == 1 else [int(v) for v in t]

    def generate_pipelined(self, prompt, steps):
        """Greedy tokens with the sampled token fed back on the device and read one step behind:
        the host records and issues step t+1 while the device still runs step t.  Per step an int, or -
        prompts of shape [B, S] - the list of the B rows' tokens."""
        tok, _ = self.prefill(prompt)
        self.be.prefetch(tok)
        toks, prev = [], tok
        for _ in range(steps - 1):
            tok, _ = self.step(prev)
            self.be.prefetch(tok)
            toks.append(self._host_tokens(prev))
            prev = tok
        toks.append(self._host_tokens(prev))
        return toks

    def generate(self, prompt, steps):
        """Returns (tokens, logits per step as numpy), reading every token before the next step like
        the reference's loop.  Per step an int, or - prompts of shape [B, S] - the list of the B rows' tokens."""
        tok, logits = self.prefill(prompt)
        toks, lg = [], []
        for _ in range(steps):
            t = self._host_tokens(tok)
            toks.append(t)
            lg.append(self.be.to_vec(logits))
            tok, logits = self.step(t)
        return toks, lg
