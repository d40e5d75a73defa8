"""Small Kegetar configurations for the tests: they differ from each other in every size and option."""
import plain_kegetar as P

KEG = {
    # both kinds of layer, both kinds of feed-forward, layers that run an earlier layer's weights
    "A": (P.make_config(vocab=97, width=64, layers=[
        P.parallel_layer(),
        P.parallel_layer(left=P.left_sizes(heads=4, kv_heads=4, dim=16, vdim=16, window=17, keep_first=5, rot_dims=8),
                         right=P.right_sizes(heads=2, dim=8, vdim=16, tau=2.0), mlp=P.experts_mlp()),
        P.attention_layer(),
        P.attention_layer(heads=2, kv_heads=2, dim=24, window=9, mlp=P.experts_mlp(ff=16, experts=5, top=3, identity=1, groups=(3, 2), shared=None)),
        P.parallel_layer(weights_of=0),
        P.attention_layer(heads=2, kv_heads=2, dim=24, window=9, mlp=P.experts_mlp(ff=16, experts=5, top=3, identity=1, groups=(3, 2), shared=None),
                          weights_of=3),
    ]), 11),
    # sizes that are no multiple of 8 or 16, one head, no pair table, no stretched frequencies, a window of one, no window at all,
    # more kept positions than the window is wide, kept positions beyond a block of 64 keys
    "B": (P.make_config(vocab=61, width=40, eps=1e-6, mult=1.3, bigram=None, layers=[
        P.attention_layer(heads=1, kv_heads=1, dim=12, window=1, mlp=None),
        P.parallel_layer(left=P.left_sizes(heads=2, kv_heads=1, dim=12, vdim=20, window=5, keep_first=9, rot_dims=6, scaling=None),
                         right=P.right_sizes(heads=1, dim=20, vdim=12, tau=1.0, decay_rank=3), mlp=P.dense_mlp(ff=20)),
        P.parallel_layer(left=P.left_sizes(heads=3, kv_heads=3, dim=8, vdim=8, window=None, rot_dims=0),
                         right=P.right_sizes(heads=3, dim=8, vdim=8, tau=30.0, decay_rank=1),
                         mlp=P.experts_mlp(ff=12, experts=4, top=1, identity=0, groups=None, limit=0.5, shared=12, shared_limit=3.0)),
        P.parallel_layer(left=P.left_sizes(heads=2, kv_heads=2, dim=16, vdim=16, window=30, keep_first=70, rot_dims=16,
                                           scaling={"factor": 8.0, "original": 16, "fast": 4.0, "slow": 2.0}),
                         right=P.right_sizes(heads=2, dim=12, vdim=4, tau=4.0, decay_rank=2), mlp=None),
        P.attention_layer(heads=6, kv_heads=2, dim=8, window=None, mlp=P.dense_mlp(ff=9)),
    ]), 21),
    # one layer; every expert chosen; the multiplier and the hash's factors equal to one
    "C": (P.make_config(vocab=33, width=32, mult=1.0, bigram=(7, 1, 1), layers=[
        P.parallel_layer(left=P.left_sizes(heads=2, kv_heads=1, dim=32, vdim=16, window=64, keep_first=1, rot_dims=32),
                         right=P.right_sizes(heads=2, dim=16, vdim=32, tau=16.0, decay_rank=8),
                         mlp=P.experts_mlp(ff=8, experts=2, top=3, identity=1, groups=None, shared=None)),
    ]), 13),
    # a width that is no multiple of 8, a vocabulary smaller than the width's square root would suggest, a layer that runs the weights of a
    # layer that runs another's
    "D": (P.make_config(vocab=50, width=36, bigram=(13, 2, 9), layers=[
        P.parallel_layer(left=P.left_sizes(heads=2, kv_heads=1, dim=16, vdim=8, window=12, keep_first=2, rot_dims=4),
                         right=P.right_sizes(heads=1, dim=8, vdim=8, tau=5.0, decay_rank=2), mlp=P.experts_mlp(ff=10, experts=3, top=2, identity=1, groups=(2, 2), shared=6)),
        P.attention_layer(heads=2, kv_heads=1, dim=8, window=6, mlp=P.dense_mlp(ff=14)),
        P.parallel_layer(left=P.left_sizes(heads=2, kv_heads=1, dim=16, vdim=8, window=12, keep_first=2, rot_dims=4),
                         right=P.right_sizes(heads=1, dim=8, vdim=8, tau=5.0, decay_rank=2), mlp=P.experts_mlp(ff=10, experts=3, top=2, identity=1, groups=(2, 2), shared=6),
                         weights_of=0),
        P.parallel_layer(left=P.left_sizes(heads=2, kv_heads=1, dim=16, vdim=8, window=12, keep_first=2, rot_dims=4),
                         right=P.right_sizes(heads=1, dim=8, vdim=8, tau=5.0, decay_rank=2), mlp=P.experts_mlp(ff=10, experts=3, top=2, identity=1, groups=(2, 2), shared=6),
                         weights_of=2),
    ]), 14),
}
