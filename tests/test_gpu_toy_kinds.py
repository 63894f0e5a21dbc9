"""Kinds of parts the framework does not have, defined here and registered from the outside: a mixer whose cache is
of a kind of its own (one latent vector a token, in pages, through a CacheSpec defined in this file), a position
encoding that is no rotation (learned vectors added to q and k, with tensors of its own in the weight file), and
a mixer with per-request state that says it may be captured, so that decode steps of its model replay HIP graphs
(padded rows of a graph use the spare state slot). No file of the framework changes for any of them; none of
them is anyone's model."""
import random
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu

LATENT, HEAD = 12, 16


def register_kinds():
    from dinfer_amd.config import ModelConfig, key, register_architecture
    from dinfer_amd.parts import (MIXERS, POSITION_ENCODINGS, CacheSpec, LayerSpec, Mixer, ModelSpec, PositionEncoding,
                                  RunEntry, StateSpec, TensorSpec, part)

    @dataclass(frozen=True)
    class LatentSpec(CacheSpec):
        """One vector of `dim` numbers a token, in pages [blocks, page, dim]."""
        dim: int

        def group_key(self):
            return ("latent", self.dim)

        def page_bytes(self, page_size, dtype):
            return page_size * self.dim * torch.empty((), dtype=dtype).element_size()

        def allocate(self, num_blocks, page_size, num_slots, dtype, device):
            return {"latent": torch.zeros((num_blocks, page_size, self.dim), dtype=dtype, device=device)}

    class LatentMixer(Mixer):
        """c_t = x_t Wc (kept in the cache), q_t = x_t Wq; y_t = softmax_j<=t(q_t . c_j / sqrt(dim)) c_j Wo^T."""

        def __init__(self, hidden, dim):
            self.hidden, self.dim = hidden, dim

        def cache_spec(self):
            return LatentSpec(self.dim)

        def tensors(self):
            return {"wc.weight": TensorSpec((self.dim, self.hidden)), "wq.weight": TensorSpec((self.dim, self.hidden)),
                    "wo.weight": TensorSpec((self.hidden, self.dim))}

        def load(self, get):
            self.wc, self.wq, self.wo = (get(n + ".weight", compute=True).float() for n in ("wc", "wq", "wo"))

        def bind(self, ctx):
            self.out = ctx.workspace.buffer("latent_out", self.hidden)
            self.page = ctx.page_size

        def forward(self, x, batch, cache):
            T, g = batch.num_tokens, cache.group
            xf = x[:T].float()
            pages = cache.latent.view(-1, self.dim)
            pages[batch.slot_mapping[g][:T]] = (xf @ self.wc.T).to(pages.dtype)     # written before anything reads
            q = xf @ self.wq.T
            table = batch.block_table[g].tolist()
            t = 0
            for b, (n, seq) in enumerate(zip(batch.q_lens, batch.seq_lens[:batch.num_reqs].tolist())):
                rows = torch.tensor([table[b][j // self.page] * self.page + j % self.page for j in range(seq)],
                                    device=x.device)
                c = pages[rows].float()                                              # the request's latents, in order
                s = (q[t:t + n] @ c.T) / self.dim ** 0.5
                first = seq - n                                                      # position of this step's first token
                hidden = torch.arange(seq, device=x.device)[None, :] > (first + torch.arange(n, device=x.device))[:, None]
                p = torch.softmax(s.masked_fill(hidden, float("-inf")), dim=-1)
                self.out[t:t + n] = ((p @ c) @ self.wo.T).to(self.out.dtype)
                t += n
            return self.out

    class LearnedPosition(PositionEncoding):
        """q += Pq[position], k += Pk[position]: vectors from the weight file, the same for every head."""
        fused = False

        def __init__(self, head_dim, max_positions):
            self.head_dim, self.max_positions = head_dim, max_positions

        def tensors(self):
            return {"q.weight": TensorSpec((self.max_positions, self.head_dim)),
                    "k.weight": TensorSpec((self.max_positions, self.head_dim))}

        def load(self, get):
            self.pq, self.pk = get("q.weight"), get("k.weight")

        def transform(self, q, k, positions):
            idx = positions.long()
            q += self.pq[idx][:, None, :].to(q.dtype)
            k += self.pk[idx][:, None, :].to(k.dtype)

    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + x_t per request (float32 state in its slot); y_t = s_t W^T. Steps of single rows
        read their slots on the device and update all states at once, so they may be captured."""
        capturable = True

        def __init__(self, hidden, decay):
            self.hidden, self.decay = hidden, decay

        def cache_spec(self):
            return StateSpec((self.hidden,), "float32")

        def tensors(self):
            return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

        def load(self, get):
            self.w = get("mix.weight", compute=True).float()

        def bind(self, ctx):
            self.out = ctx.workspace.buffer("decay_out", self.hidden)

        def forward(self, x, batch, cache):
            B, T = batch.num_reqs, batch.num_tokens
            if batch.all_decode:
                slots = batch.state_slots[:B].long()            # on the device: a replay brings other slots
                s = cache.state[slots] * self.decay + x[:B].float()
                cache.state.index_copy_(0, slots, s)
                self.out[:B] = (s @ self.w.T).to(self.out.dtype)
                return self.out
            t = 0
            for slot, n in zip(batch.state_slots[:B].tolist(), batch.q_lens):
                s = cache.state[slot]
                for i in range(n):
                    s.mul_(self.decay).add_(x[t + i].float())
                    self.out[t + i] = (s @ self.w.T).to(self.out.dtype)
                t += n
            return self.out

    @dataclass(frozen=True)
    class KindsConfig(ModelConfig):
        vocab_size: int = key(int)
        hidden_size: int = key(int)
        decay: float = key(float)
        latent: bool = key(bool, True)
        ARCHITECTURE = "ToyKindsLM"

    def build_spec(c):
        norm = part("rmsnorm", eps=1e-5)
        ff = part("gated_mlp", intermediate=40)
        learned = part("toy_learned_position", max_positions=96)
        layers = [LayerSpec(part("prenorm", mixer_prefix="latent."), part("toy_latent", dim=LATENT), ff, norm, "layers.0."),
                  LayerSpec(part("prenorm"), part("attention", heads=2, kv_heads=1, head_dim=HEAD, position=learned,
                                                  qk_norm=part("rmsnorm", eps=1e-5)), ff, norm, "layers.1."),
                  LayerSpec(part("prenorm", mixer_prefix="decay."), part("toy_decay_vec", decay=c.decay), ff, norm, "layers.2.")]
        run = [RunEntry(0), RunEntry(1), RunEntry(2)] if c.latent else [RunEntry(1), RunEntry(2)]
        return ModelSpec("ToyKindsLM", c.vocab_size, c.hidden_size, 96, layers if c.latent else layers, run, norm, "norm.",
                         "embed.weight", "head.weight", tie_embeddings=True)

    MIXERS.register("toy_latent", LatentMixer)
    MIXERS.register("toy_decay_vec", DecayMixer)
    POSITION_ENCODINGS.register("toy_learned_position", LearnedPosition)
    register_architecture("ToyKindsLM", KindsConfig, build_spec)
    return KindsConfig


def unregister_kinds():
    from dinfer_amd.config import unregister_architecture
    from dinfer_amd.parts import MIXERS, POSITION_ENCODINGS
    unregister_architecture("ToyKindsLM")
    MIXERS.unregister("toy_latent")
    MIXERS.unregister("toy_decay_vec")
    POSITION_ENCODINGS.unregister("toy_learned_position")


def kinds_plain(w, ids, decay, latent=True):
    """The toy model for one whole sequence, straight torch in float64."""
    W = {k: v.double() for k, v in w.items()}
    T = len(ids)
    h = W["embed.weight"][ids]
    eps = 1e-5

    def ffn(p, x):
        return plain.swiglu_mlp(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])

    def latent_layer(h):
        p = "layers.0."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], eps)
        c, q = x @ W[p + "latent.wc.weight"].T, x @ W[p + "latent.wq.weight"].T
        s = (q @ c.T) / LATENT ** 0.5
        s = s.masked_fill(torch.arange(T)[None, :] > torch.arange(T)[:, None], float("-inf"))
        h = h + (torch.softmax(s, -1) @ c) @ W[p + "latent.wo.weight"].T
        return h + ffn(p, plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))

    def attn_layer(h):
        p = "layers.1."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], eps)
        q = plain.rms_norm((x @ W[p + "self_attn.q_proj.weight"].T).view(T, 2, HEAD), W[p + "self_attn.q_norm.weight"], eps)
        k = plain.rms_norm((x @ W[p + "self_attn.k_proj.weight"].T).view(T, 1, HEAD), W[p + "self_attn.k_norm.weight"], eps)
        v = (x @ W[p + "self_attn.v_proj.weight"].T).view(T, 1, HEAD)
        q = q + W[p + "self_attn.position.q.weight"][:T, None, :]
        k = k + W[p + "self_attn.position.k.weight"][:T, None, :]
        h = h + plain.causal_attention(q, k, v, HEAD ** -0.5).reshape(T, 2 * HEAD) @ W[p + "self_attn.o_proj.weight"].T
        return h + ffn(p, plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))

    def decay_layer(h):
        p = "layers.2."
        x = plain.rms_norm(h, W[p + "input_layernorm.weight"], eps)
        s, ys = torch.zeros(h.shape[1], dtype=torch.float64), []
        for t in range(T):
            s = decay * s + x[t]
            ys.append(s @ W[p + "decay.mix.weight"].T)
        h = h + torch.stack(ys)
        return h + ffn(p, plain.rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))

    if latent:
        h = latent_layer(h)
    h = decay_layer(attn_layer(h))
    return plain.rms_norm(h, W["norm.weight"], eps) @ W["embed.weight"].T


def run_plan(r, plan, seqs, want, fed):
    """plan: steps of [(request, tokens this step)]; every row against the plain logits; requests that end are freed."""
    from dinfer_amd.engine.batch import Entry
    for st in plan:
        entries = []
        for k, n in st:
            assert r.reserve(k, fed[k], n)
            entries.append(Entry(k, seqs[k][fed[k]:fed[k] + n], fed[k], list(range(n))))
        logits = r.step(entries).double().cpu()
        i = 0
        for e in entries:
            n = len(e.tokens)
            torch.testing.assert_close(logits[i:i + n], want[e.req_id][e.start:e.start + n], rtol=2e-4, atol=2e-5,
                                       msg=lambda m, e=e: f"request {e.req_id} at {e.start}: {m}")
            i += n
            fed[e.req_id] += n
            if fed[e.req_id] == len(seqs[e.req_id]):
                r.finish(e.req_id)
        r.cache.check()


def test_cache_kind_and_position_encoding_of_their_own(tmp_path):
    """The latent mixer's cache is allocated, grouped and paged through the CacheSpec it brings (a group beside the
    attention layer's keys and values, each with its own block table); the learned position vectors come from the
    weight file under the attention's prefix and reach the keys before they are cached."""
    from safetensors.torch import load_file
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.weights import write_random_model
    Config = register_kinds()
    try:
        cfg = Config.from_dict(dict(vocab_size=101, hidden_size=24, decay=0.7, architectures=["ToyKindsLM"]))
        write_random_model(cfg, tmp_path, seed=8, dtype="float32")
        w = load_file(str(tmp_path / "model.safetensors"))
        assert "layers.0.latent.wc.weight" in w and "layers.1.self_attn.position.k.weight" in w
        opt = EngineOptions(dtype="float32", max_model_len=96, max_num_seqs=3, max_num_batched_tokens=64, block_size=8,
                            num_blocks=14, max_logits_rows=64, decode_exempt_from_budget=False)
        r = ModelRunner.from_dir(tmp_path, opt)
        assert len(r.group_specs) == 2 and len(r.state_tensors) == 1
        assert r.cache_views[0].latent.shape == (14, 8, LATENT) and r.cache_views[0].k is None
        assert not r.cache.prefix_caching and not r._graphs_allowed     # state of its own; a mixer that reads host lists
        rng = random.Random(3)
        seqs = {k: [rng.randrange(101) for _ in range(n)] for k, n in (("a", 37), ("b", 50), ("c", 9), ("d", 30))}
        want = {k: kinds_plain(w, v, 0.7) for k, v in seqs.items()}
        fed = {k: 0 for k in seqs}
        # 14 pages of 8 hold a and b and c (5 + 7 + 2); d runs on the pages a and c gave back
        plan = [[("a", 5), ("b", 2)], [("b", 17)], [("a", 16), ("b", 1), ("c", 9)], [("a", 16), ("b", 30)], [("d", 21)],
                [("d", 1)], [("d", 8)]]
        run_plan(r, plan, seqs, want, fed)
        assert all(r.cache.num_free(g) == 14 for g in range(2))
    finally:
        unregister_kinds()


def test_state_of_its_own_under_captured_graphs(tmp_path):
    """A model whose parts all say they may be captured, one of them with per-request state: steps of single rows
    replay graphs of 1, 2 and 4 rows. With three requests the fourth row of the graph is padding; it works on the
    spare state slot and leaves the requests' states alone. A request that ends gives its slot to the next one,
    whose state starts from zero although the graph that then runs was captured while the slot held the other's."""
    from safetensors.torch import load_file
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    from dinfer_amd.weights import write_random_model
    Config = register_kinds()
    try:
        cfg = Config.from_dict(dict(vocab_size=101, hidden_size=24, decay=0.6, latent=False, architectures=["ToyKindsLM"]))
        write_random_model(cfg, tmp_path, seed=9, dtype="float32")
        w = load_file(str(tmp_path / "model.safetensors"))
        opt = EngineOptions(dtype="float32", max_model_len=96, max_num_seqs=4, max_num_batched_tokens=64, block_size=8,
                            num_blocks=40, max_logits_rows=64, decode_exempt_from_budget=False, hip_graph=True)
        r = ModelRunner.from_dir(tmp_path, opt)
        assert r._graphs_allowed and r.state_tensors[0].shape[0] == 5           # four requests and the spare slot
        rng = random.Random(5)
        lens = {"a": 30, "b": 22, "c": 41, "d": 25, "e": 18}
        seqs = {k: [rng.randrange(101) for _ in range(n)] for k, n in lens.items()}
        want = {k: kinds_plain(w, v, 0.6, latent=False) for k, v in seqs.items()}
        fed = {k: 0 for k in seqs}
        plan = [[("a", 9), ("b", 4)], [("c", 12)]]
        plan += [[("a", 1), ("b", 1), ("c", 1)]] * 10                   # three rows in the graph of four
        plan += [[("a", 1)]] * 3 + [[("a", 1), ("c", 1)]] * 4            # graphs of one and of two rows
        plan += [[("b", 8)], [("a", 4), ("c", 14)]]                      # b ends: its slot is free; a ends
        plan += [[("d", 11), ("e", 6)]]                                  # d and e take the slots of b and a
        plan += [[("d", 1), ("e", 1)]] * 12                              # graph of two rows, captured with a and c in it
        plan += [[("d", 2)]]
        run_plan(r, plan, seqs, want, fed)
        assert sorted(b for b, _ in r._graphs) == [1, 2, 4]
        assert fed["a"] == 30 and fed["b"] == 22 and fed["d"] == 25 and fed["e"] == 18
    finally:
        unregister_kinds()
