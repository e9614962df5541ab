"""The Zovozen decoder as a list of parts chosen by ZovozenConfig, layer by layer: a plain embedding; layers whose
sublayers read the residual stream itself and whose results are normed before the sum (x <- x + norm1(mixer(x)), then
x <- x + norm2(ff(x))); a mixer of two side by side, a_left left + a_right right: on the left softmax attention whose
scores are mixed over the heads before the softmax (biases, queries and keys normed over the whole projection, rotary
positions on part of a head with linear scaling, values normed per head, a temperature and a sink a head, blocks of
positions that see only themselves, an output gate), on the right a matrix memory with exponential gates (mLSTM);
feed-forwards that are dense (squared relu, biases) or a mixture of gated experts routed by softmax scores with a
correction for the choice, groups, identity experts and a shared expert; the logits are the embedding table times the
normed last rows.  Tensor names: `embed`, `l<i>.norm1|norm2`, `l<i>.mix.left.*`, `l<i>.mix.right.*`,
`l<i>.mlp.up|down(.b)` or `l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down`, `final.norm`.
"""
from ..config.base import register_architecture
from ..config.zovozen import ZovozenConfig
from ..parts import make_part, LMHead, PairHashEmbedding
from .model import Model


def build_zovozen(config):
    c = config
    H, eps = c.width, c.norm_eps

    def norm(tensor):
        return make_part("norm", "rmsnorm", name=tensor, dim=H, eps=eps, tensor=tensor)

    positions = {}

    def position(a):
        # one part (one pair of tables) for all layers that turn alike
        key = (a.rot, a.dim)
        if key not in positions:
            if a.rot is None:
                positions[key] = make_part("position", "none", head_dim=a.dim, max_positions=1)
            else:
                positions[key] = make_part("position", "rotary", head_dim=a.dim, theta=a.rot.base, max_positions=c.max_positions,
                                           rotary_dim=a.rot.dims, pairing="split_half",
                                           scaling=None if a.rot.factor == 1.0 else {"factor": a.rot.factor})
        return positions[key]

    layers = []
    for i, spec in enumerate(c.layers):
        p, a, r = f"l{i}", spec.mixer.left, spec.mixer.right
        left = make_part("mixer", "talking_attention", name=p + ".mix.left", hidden=H, heads=a.heads, kv_heads=a.kv_heads, dim=a.dim,
                         vdim=a.vdim, scale=a.scale, eps=eps, position=position(a), chunk=a.chunk)
        right = make_part("mixer", "matrix_memory", name=p + ".mix.right", hidden=H, heads=r.heads, dim=r.dim, vdim=r.vdim,
                          gate_cap=r.gate_cap, eps=eps)
        mixer = make_part("mixer", "side_by_side", name=p + ".mix", hidden=H, first=left, second=right, eps=eps,
                          scales=(spec.mixer.left_scale, spec.mixer.right_scale))
        ffn = {}
        m = spec.mlp
        if m is not None and m.kind == "dense":
            ffn = dict(ffn=make_part("ffn", "dense_mlp", name=p + ".mlp", hidden=H, intermediate=m.ff, activation="relu2", bias=True),
                       ffn_post=norm(p + ".norm2"))
        elif m is not None:
            shared = None
            if m.shared_ff is not None:
                shared = make_part("ffn", "gated_mlp", name=p + ".mlp.shared", hidden=H, intermediate=m.shared_ff, names=("gate", "up", "down"))
            ffn = dict(ffn=make_part("ffn", "scored_experts", name=p + ".mlp", hidden=H, intermediate=m.ff, experts=m.experts, top=m.top,
                                     identity=m.identity, groups=m.groups, shared=shared),
                       ffn_post=norm(p + ".norm2"))
        layers.append(make_part("block", "sandwich", mixer_norm=None, mixer=mixer, mixer_post=norm(p + ".norm1"), reads_stream=True, **ffn))
    embedding = PairHashEmbedding("embed", c.vocab, H, tensor="embed")
    head = LMHead("head", c.vocab, H, tied_to=embedding)
    return Model(c, embedding, layers, norm("final.norm"), head, max_positions=c.max_positions, vocab_size=c.vocab)


register_architecture(["Zovozen", "zovozen"], ZovozenConfig, build_zovozen)
