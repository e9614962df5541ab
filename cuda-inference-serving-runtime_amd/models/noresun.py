"""The Noresun decoder as a list of parts chosen by NoresunConfig, layer by layer: an embedding times a scale plus a
table of hashed token pairs; layers that norm after the sum (x <- norm(alpha x + gate * sublayer(x)), the sublayers
reading x itself, each result gated element by element by sigmoid(W x + b)); a mixer that is attention with sigmoid
weights (no softmax; queries and keys normed over the whole projection, neighbouring rotary pairs with frequencies
scaled by wavelength, a sliding window, a bias a head; optionally reading the keys and values of an earlier layer) or
a minimal gated recurrent unit; feed-forwards of routed experts with squared-relu units; the logits are the embedding
table (without its scale) times the normed last rows.  Tensor names: `embed`, `bigram`, `l<i>.norm1|norm2`,
`l<i>.rg1|rg2(.b)`, `l<i>.mix.*`, `l<i>.mlp.router(.b)`, `l<i>.mlp.e<j>.up|down`, `final.norm`.
"""
from ..config.base import register_architecture
from ..config.noresun import NoresunConfig
from ..parts import make_part, LMHead, PairHashEmbedding
from .model import Model, ScheduleEntry


def build_noresun(config):
    c = config
    H, eps = c.width, c.norm_eps

    def norm(tensor):
        return make_part("norm", "rmsnorm", name=tensor, dim=H, eps=eps, tensor=tensor)

    positions = {}

    def position(a):
        # one part (one pair of tables) for all layers that turn alike
        if a.rot not in positions:
            scaling = None if a.rot.scaling is None else dict(zip(("factor", "low", "high", "original"), a.rot.scaling))
            positions[a.rot] = make_part("position", "rotary", head_dim=a.rot.dims, theta=a.rot.base, max_positions=c.max_positions,
                                         rotary_dim=a.rot.dims, pairing="interleaved", scaling=scaling)
        return positions[a.rot]

    # a layer whose keys others read keeps as many as the one of them that looks back furthest
    keep = {}
    for i, spec in enumerate(c.layers):
        a = spec.attention
        if a is not None:
            source = i if a.kv_from is None else a.kv_from
            windows = keep.setdefault(source, [])
            windows.append(a.window)
    keep = {i: None if None in windows else max(windows) for i, windows in keep.items()}

    layers, schedule = [], []
    for i, spec in enumerate(c.layers):
        p = f"l{i}"
        if spec.type == "mingru":
            mixer = make_part("mixer", "mingru", name=p + ".mix", hidden=H, width=spec.mingru.width)
            schedule.append(ScheduleEntry(i))
        else:
            a = spec.attention
            own = a.kv_from is None
            mixer = make_part("mixer", "sigmoid_attention", name=p + ".mix", hidden=H, heads=a.heads, kv_heads=a.kv_heads, dim=a.dim,
                              vdim=a.vdim, scale=a.scale, eps=eps, position=position(a), window=a.window,
                              keep=keep[i] if own else "own", own_kv=own)
            schedule.append(ScheduleEntry(i, reads=None if own else a.kv_from))
        ffn = {}
        if spec.mlp is not None:
            m = spec.mlp
            ffn = dict(ffn_norm=norm(p + ".norm2"),
                       ffn=make_part("ffn", "routed_experts", name=p + ".mlp", hidden=H, intermediate=m.ff, experts=m.experts, top=m.top))
        layers.append(make_part("block", "postnorm", name=p, hidden=H, mixer_norm=norm(p + ".norm1"), mixer=mixer, alpha=c.postln_alpha,
                                gated=True, **ffn))
    b = c.bigram
    embedding = PairHashEmbedding("embed", c.vocab, H, scale=c.embedding_scale, tensor="embed", pairs_tensor="bigram",
                                  **({} if b is None else dict(buckets=b.buckets, mul_prev=b.mul_prev, mul_cur=b.mul_cur)))
    head = LMHead("head", c.vocab, H, tied_to=embedding)
    return Model(c, embedding, layers, norm("final.norm"), head, schedule=schedule, max_positions=c.max_positions, vocab_size=c.vocab)


register_architecture(["Noresun", "noresun"], NoresunConfig, build_noresun)
