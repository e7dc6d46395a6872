"""One decoding step of a Marian transformer decoder on the HIP library, through the host mirrors
(integer.py, ops.py): the embedding of the previous step's words (reference
src/models/transformer.h:92-117: rows of the table times sqrt(d), plus the position signal), the
call sequence of reference src/models/transformer.h:603-760 for one new target position at
inference (post-processing "dan": skip connection, then layer norm), followed by
the log-softmax and the beam search's n-best selection (src/translator/beam_search.cpp:472-492).
Weights are random; the key/value caches of earlier target positions and of the encoder are
resident.  bench.py times it at transformer-big size; tests check every call of it against the CPU
checker."""
import torch

from . import integer, ops


class DecoderStep:
    """Transformer-big decoder (6 layers, d = 1024, ffn = 4096, 16 heads, tied 32000-word output
    layer) with random-init weights, driven through the host mirrors of the library: one full
    decoding step at beam 4 x batch 32 (reference src/models/transformer.h:603-760 for the layer
    structure, post-processing "dan", inference).  Self-attention keys/values of `t_past` earlier
    positions and encoder keys/values of `src_len` positions are resident; K/V projections are
    taken for the new position only.  The step starts from the word indices the previous step
    chose (the float32 embedding table is the transposed output matrix: tied embeddings, which
    intgemm models keep in float32, reference src/tensors/cpu/expression_graph_packable.h:154).
    Beam search's hypothesis bookkeeping is not part of the step."""

    def __init__(self, sets=1, d=1024, ffn=4096, heads=16, vocab=32000, layers=6, beam=4, batch=32,
                 t_past=20, src_len=60, min_src_len=20, seed=300, t_capacity=None, ancestors=False):
        self.torch, self.integer, self.ops = torch, integer, ops
        self.d, self.ffn, self.V, self.H = d, ffn, vocab, heads
        self.beam, self.batch, self.layers = beam, batch, layers
        self.M = self.beam * self.batch
        self.T, self.L = t_past + 1, src_len   # T: cached positions in use, the step's new one included
        self.cap = self.T if t_capacity is None else int(t_capacity)   # positions the caches have room for
        assert self.cap >= self.T
        self.trace = None   # a list: every operator call of step() is recorded into it (tests)
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        d, ffn, V, H, M = self.d, self.ffn, self.V, self.H, self.M

        def qw(K, N):
            return integer.prepareB(torch.randn(K, N, device="cuda", generator=g) * 0.02)

        def vec(n, scale=0.01, shift=0.0):
            return torch.randn(n, device="cuda", generator=g) * scale + shift

        # tied embeddings: one float32 table [V, d] for the lookup, its transpose quantized for the output layer
        self.E = torch.randn(V, d, device="cuda", generator=g) * 0.02
        first = {"layers": [], "out": (integer.prepareB(self.E.t().contiguous()), vec(V))}
        for _ in range(layers):
            ly = {}
            for name, (K, N) in {"Wq": (d, d), "Wk": (d, d), "Wv": (d, d), "Wo": (d, d), "cWq": (d, d),
                                 "cWo": (d, d), "W1": (d, ffn), "W2": (ffn, d)}.items():
                ly[name] = (qw(K, N), vec(N))
            for name in ("ln1", "ln2", "ln3"):
                ly[name] = (vec(d, 0.1, 1.0), vec(d, 0.1))
            first["layers"].append(ly)

        def clone(x):
            if isinstance(x, dict):
                return {k: clone(v) for k, v in x.items()}
            if isinstance(x, (list, tuple)):
                return type(x)(clone(v) for v in x)
            if isinstance(x, integer.QTensor):
                return integer.QTensor(x.data.clone(), x.shape, x.type, x.prepared)
            return x   # small fp32 vectors are shared
        self.sets = [first] + [clone(first) for _ in range(sets - 1)]
        self.weight_bytes = layers * (6 * d * d + 2 * d * ffn) + d * V
        self.gemm_ops = 2 * M * self.weight_bytes
        # resident state
        self.words = torch.randint(0, V, (M,), device="cuda", generator=g).to(torch.int32)
        self.signal = ops.sinusoidalPositionEmbeddings(1, d, t_past, device="cuda")
        self.emb_scale = float(torch.sqrt(torch.tensor(float(d))))
        self.x = torch.randn(M, d, device="cuda", generator=g)   # (input of the GEMM-only chain)
        # the self-attention caches of all layers are rows of one tensor [2 * layers * M, H * cap * dk] (a
        # hypothesis's cached positions of one layer are one row), so that the beam search's selection
        # of the surviving hypotheses is one gather; a second tensor of that size receives it
        self.state = torch.randn(2 * layers * M, H * self.cap * (d // H), device="cuda", generator=g)
        self.state_next = torch.empty_like(self.state)
        self._cache_views()
        # back-pointers of a beam-search step: hypothesis (k, b) continues hypothesis (k', b) of the
        # same sentence; flat index k * batch + b, one copy per cache tensor
        parent = torch.randint(0, beam, (beam, batch), device="cuda", generator=g) * batch + torch.arange(batch, device="cuda")
        self.set_hypotheses(parent.reshape(-1))
        # ancestors: the caches are never moved; a table says in whose entry a position of a
        # hypothesis's history lies (at the start: in its own), and the state selection rewrites the table
        self.by_ancestors = bool(ancestors)
        if self.by_ancestors:
            self.anc = torch.arange(M, device="cuda", dtype=torch.int32)[:, None].repeat(1, self.cap).contiguous()
            self.anc_next = torch.empty_like(self.anc)
        self.Kenc = [torch.randn(self.batch * H, self.L, d // H, device="cuda", generator=g) for _ in range(layers)]
        self.Venc = [torch.randn(self.batch * H, self.L, d // H, device="cuda", generator=g) for _ in range(layers)]
        # source lengths uniform over min_src_len .. src_len, padded to the longest (the mask covers the rest)
        lens = torch.randint(min_src_len, self.L + 1, (self.batch,), device="cuda", generator=g)
        self.src_lens = lens
        self.mask = (torch.arange(self.L, device="cuda")[None, :] >= lens[:, None]).float() * -99999999.0

    def _cache_views(self):
        M, H, cap, dk, layers = self.M, self.H, self.cap, self.d // self.H, self.layers
        self.Kself = [self.state[l * M:(l + 1) * M].view(M * H, cap, dk) for l in range(layers)]
        self.Vself = [self.state[(layers + l) * M:(layers + l + 1) * M].view(M * H, cap, dk) for l in range(layers)]

    def set_hypotheses(self, hyp_indices):
        """back-pointers of the next step: hypothesis i continues hypothesis hyp_indices[i] (flat
        index beam entry * batch + sentence), one copy per cache tensor for the gather"""
        self.hyp_indices = hyp_indices.to(device="cuda", dtype=torch.int32).contiguous()
        self.state_rows = (torch.arange(2 * self.layers, device="cuda", dtype=torch.int32)[:, None] * self.M +
                           self.hyp_indices[None, :]).reshape(-1).contiguous()

    def advance(self, words, hyp_indices):
        """The next target position: the words the beam search chose, the hypotheses they continue
        (step(select=True) then gathers their caches), one more cached position in use."""
        assert self.T < self.cap, "the caches are full"
        self.words = words.to(device="cuda", dtype=torch.int32).contiguous()
        self.set_hypotheses(hyp_indices)
        self.T += 1
        self.signal = self.ops.sinusoidalPositionEmbeddings(1, self.d, self.T - 1, device="cuda")

    def select_states(self):
        """The decoder state of the surviving hypotheses (reference src/models/states.h:87-107,
        src/rnn/types.h:22-42: rows(state, hypIndices) per cached tensor) for all layers in one
        gather; the two state tensors swap roles."""
        if self.by_ancestors:
            self.ops.advanceAncestors(self.anc, self.hyp_indices, self.T - 1, self.anc_next)
            self.anc, self.anc_next = self.anc_next, self.anc
            return
        H, span = self.H, self.cap * (self.d // self.H)
        # (the positions cached so far: the step's own position is appended behind them afterwards)
        self.ops.selectState(self.state.view(-1, H, span), self.state_rows, self.state_next.view(-1, H, span),
                             used=(self.T - 1) * (self.d // self.H))
        self.state, self.state_next = self.state_next, self.state
        self._cache_views()

    def step(self, s, gemm_only=False, chained=True, grouped=True, fused_tail=False, select=False, fused_attention=True):
        """chained: every tensor that feeds an affine call leaves its abs-max where it is
        produced (layer norm, attention, the ReLU GEMM), so those calls skip their abs-max pass.
        grouped: the self-attention projections Wq, Wk, Wv (one input, three weight matrices,
        reference src/models/transformer.h:290-325) go through one call.
        fused_tail: log-softmax and n-best in one launch (the log-probabilities are not written);
        the step then returns (scores, keys) of the n-best instead of the log-probabilities.
        select: the step starts with the selection of the surviving hypotheses' cached keys and
        values by the back-pointers self.hyp_indices, as a beam-search step does.
        fused_attention: the projections in front of an attention (Wq, Wk, Wv; the context
        attention's Wq) and the attention itself are one launch each (ops.ProjectedAttention)."""
        integer, ops = self.integer, self.ops
        W = self.sets[s % len(self.sets)]
        tr = self.trace

        def rec(kind, **kw):   # clones: later calls overwrite nothing, but the caches are updated in place
            if tr is not None:
                tr.append((kind, {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}))
        H, M, d = self.H, self.M, self.d
        dk = d // H
        x, xmax = self.x, None
        ch = chained and not gemm_only
        if select and not gemm_only:
            before = self.state
            self.select_states()
            if not self.by_ancestors:
                rec("select", state=before, rows=self.state_rows, out=self.state, heads=H, used=(self.T - 1) * dk)
        if not gemm_only:
            x = ops.scaledEmbeddings(self.E, self.words, self.emb_scale, self.signal, M, want_absmax=ch)
            if ch:
                x, xmax = x
            rec("embed", E=self.E, ids=self.words, scale=self.emb_scale, signal=self.signal, out=x, position=self.T - 1)
        for li, ly in enumerate(W["layers"]):
            omax = x1max = comax = x2max = f1max = None
            fuse = fused_attention and not gemm_only and not self.by_ancestors and ch
            if fuse:   # q, k, v and the self-attention over the cache (the new position appended) in one launch
                if tr is not None:
                    k_before, v_before = self.Kself[li].clone(), self.Vself[li].clone()
                res = ops.ProjectedAttention(x, [ly["Wq"], ly["Wk"], ly["Wv"]], self.Kself[li], self.Vself[li], H,
                                             kvLen=self.T, absmax=xmax, want_absmax=True, want_projections=tr is not None)
                o, omax = res[0], res[2]
                if tr is not None:
                    q, k, v = res[3]
                    for name, t in (("Wq", q), ("Wk", k), ("Wv", v)):
                        rec("affine", a=x, w=ly[name], out=t, relu=False)
                    rec("self_attention", q=q, k_new=k, v_new=v, k_cache=k_before, v_cache=v_before,
                        k_after=self.Kself[li], v_after=self.Vself[li], out=o, len=self.T)
                o = o.view(M, d)
            else:
                if grouped:   # one abs-max, one quantization, one launch for the three projections
                    (q, k, v), _ = integer.affine_f32_grouped(x, [ly["Wq"], ly["Wk"], ly["Wv"]], absmax=xmax)
                else:
                    q, _ = integer.affine_f32(x, *ly["Wq"], absmax=xmax)
                    k, _ = integer.affine_f32(x, *ly["Wk"], absmax=xmax)
                    v, _ = integer.affine_f32(x, *ly["Wv"], absmax=xmax)
                for name, t in (("Wq", q), ("Wk", k), ("Wv", v)):
                    rec("affine", a=x, w=ly[name], out=t, relu=False)
                if gemm_only:
                    o = q
                else:
                    # head split of a single position is a view; the attention call also appends the
                    # new key/value to the cache
                    if tr is not None:
                        k_before, v_before = self.Kself[li].clone(), self.Vself[li].clone()
                    if self.by_ancestors:
                        o = ops.AttentionByAncestors(q.view(M * H, 1, dk), self.Kself[li], self.Vself[li], self.anc, self.T,
                                                     k.view(M * H, dk), v.view(M * H, dk), want_absmax=ch)
                    else:
                        o = ops.Attention(q.view(M * H, 1, dk), self.Kself[li], self.Vself[li], want_absmax=ch,
                                          kNew=k.view(M * H, dk), vNew=v.view(M * H, dk), kvLen=self.T)
                    if ch:
                        o, omax = o
                    if tr is not None:
                        rec("self_attention", q=q, k_new=k, v_new=v, k_cache=k_before, v_cache=v_before,
                            k_after=self.Kself[li], v_after=self.Vself[li], out=o, len=self.T)
                    o = o.view(M, d)
            a, _ = integer.affine_f32(o, *ly["Wo"], absmax=omax)
            rec("affine", a=o, w=ly["Wo"], out=a, relu=False)
            if gemm_only:
                x1 = a
            else:
                x1 = ops.layerNorm(a, *ly["ln1"], eps=1e-6, add=x, want_absmax=ch)
                if ch:
                    x1, x1max = x1
                rec("layer_norm", x=a, add=x, gamma=ly["ln1"][0], beta=ly["ln1"][1], out=x1)
            if fused_attention and not gemm_only and ch:   # the context attention's Wq and the attention in one launch
                res = ops.ProjectedAttention(x1, [ly["cWq"]], self.Kenc[li], self.Venc[li], H, mask=self.mask,
                                             absmax=x1max, want_absmax=True, want_projections=tr is not None)
                co, comax = res[0], res[2]
                if tr is not None:
                    cq = res[3][0]
                    rec("affine", a=x1, w=ly["cWq"], out=cq, relu=False)
                    rec("context_attention", q=cq, k=self.Kenc[li], v=self.Venc[li], mask=self.mask, out=co)
                co = co.view(M, d)
            else:
                cq, _ = integer.affine_f32(x1, *ly["cWq"], absmax=x1max)
                rec("affine", a=x1, w=ly["cWq"], out=cq, relu=False)
                if gemm_only:
                    co = cq
                else:
                    co = ops.Attention(cq.view(M * H, 1, dk), self.Kenc[li], self.Venc[li], self.mask,
                                       rowsPerMask=H, want_absmax=ch)
                    if ch:
                        co, comax = co
                    rec("context_attention", q=cq, k=self.Kenc[li], v=self.Venc[li], mask=self.mask, out=co)
                    co = co.view(M, d)
            ca, _ = integer.affine_f32(co, *ly["cWo"], absmax=comax)
            rec("affine", a=co, w=ly["cWo"], out=ca, relu=False)
            if gemm_only:
                x2 = ca
            else:
                x2 = ops.layerNorm(ca, *ly["ln2"], eps=1e-6, add=x1, want_absmax=ch)
                if ch:
                    x2, x2max = x2
                rec("layer_norm", x=ca, add=x1, gamma=ly["ln2"][0], beta=ly["ln2"][1], out=x2)
            f1 = integer.affine_f32(x2, *ly["W1"], relu=True, absmax=x2max, want_absmax=ch)
            if ch:
                f1, _, f1max = f1
            else:
                f1 = f1[0]
            rec("affine", a=x2, w=ly["W1"], out=f1, relu=True)
            f2, _ = integer.affine_f32(f1, *ly["W2"], absmax=f1max)
            rec("affine", a=f1, w=ly["W2"], out=f2, relu=False)
            if gemm_only:
                x = f2
            else:
                xin = x2
                x = ops.layerNorm(f2, *ly["ln3"], eps=1e-6, add=x2, want_absmax=ch)
                if ch:
                    x, xmax = x
                rec("layer_norm", x=f2, add=xin, gamma=ly["ln3"][0], beta=ly["ln3"][1], out=x)
        logits, _ = integer.affine_f32(x, *W["out"], absmax=xmax)
        rec("affine", a=x, w=W["out"], out=logits, relu=False)
        if gemm_only:
            return logits
        if fused_tail:
            vals, keys = ops.logsoftmaxNBestOfBeams(logits.view(self.beam, 1, self.batch, self.V), self.beam)
            rec("logsoftmax_nbest", logits=logits, vals=vals, keys=keys)
            return vals, keys
        # log-probabilities, then the beam's n-best per sentence over beam x vocabulary
        lp = ops.logsoftmax(logits)
        # (the transposition to [batch, beam * V] of beam_search.cpp:472 happens inside the call)
        vals, keys = ops.getNBestListOfBeams(lp.view(self.beam, 1, self.batch, self.V), self.beam)
        rec("logsoftmax", x=logits, out=lp)
        rec("nbest", scores=lp, vals=vals, keys=keys)
        return lp
