"""Small Tativik configurations for the tests. They differ from layer to layer and from one another in every size and
option: the order of the two kinds of layer, windows shorter and longer than a page, of exactly one page, of one position
and none, layers that read the latent of an earlier layer (with a smaller and a larger window than its owner, two readers
of one owner, a reader right behind and far behind its owner), rotations of the whole rotated part, of a piece of it and
of nothing, one head and several, sizes that are multiples of 16 and sizes that are not of 8, one to four norm groups,
routers with and without groups (one group, every group kept, fewer kept), one to three experts a token, layers without a
feed-forward."""
import plain_tativik as P

# windows of 24 and 37 straddle pages of 16; layer 1 reads layer 0's latent through a larger window, layer 3 through a smaller one
TAT_A = P.make_config(vocab=97, width=64, eps=1e-5, groups=2, mult=0.7, layers=[
    P.latent_layer(heads=4, dim=16, rot_dim=8, vdim=8, kv_rank=24, q_rank=16, window=24, base=100.0, mlp=P.experts_mlp(ff=24, experts=8, top=2, groups=(4, 2))),
    P.latent_layer(heads=2, dim=8, rot_dim=8, vdim=24, kv_rank=24, q_rank=40, window=37, base=100.0, kv_from=0, scale=0.3, mlp=None),
    P.delta_layer(heads=2, dim=16, decay_rank=8, mlp=P.experts_mlp(ff=20, experts=6, top=3)),
    P.latent_layer(heads=3, dim=16, rot_dim=8, vdim=16, kv_rank=24, q_rank=8, window=9, base=100.0, kv_from=0, mlp=P.experts_mlp(ff=16, experts=4, top=1, groups=(2, 1))),
    P.delta_layer(heads=4, dim=8, decay_rank=5, mlp=None),
])

# sizes the matrix-core kernels take (multiples of 16); a window of exactly one page; the recurrent layer first; four norm groups
TAT_B = P.make_config(vocab=211, width=96, eps=1e-6, groups=4, mult=1.3, layers=[
    P.delta_layer(heads=3, dim=32, decay_rank=16, mlp=P.experts_mlp(ff=48, experts=12, top=2, groups=(3, 3))),
    P.latent_layer(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48, q_rank=64, window=16, base=1000.0, mlp=P.experts_mlp(ff=32, experts=8, top=3, groups=(4, 3))),
    P.latent_layer(heads=2, dim=16, rot_dim=32, vdim=16, kv_rank=32, q_rank=32, window=70, rot_dims=16, base=50.0, mlp=P.experts_mlp(ff=64, experts=4, top=2)),
    P.latent_layer(heads=5, dim=16, rot_dim=32, vdim=48, kv_rank=32, q_rank=16, window=None, rot_dims=16, base=50.0, kv_from=2, mlp=None),
])

# one layer of each kind, one head, one norm group, one expert a token out of two, a window of one position (a query sees itself
# and the sink alone), no rotated part at all
TAT_C = P.make_config(vocab=50, width=32, eps=1e-3, groups=1, mult=1.0, layers=[
    P.latent_layer(heads=1, dim=8, rot_dim=0, vdim=24, kv_rank=8, q_rank=8, window=1, mlp=P.experts_mlp(ff=8, experts=2, top=1)),
    P.delta_layer(heads=1, dim=24, decay_rank=1, mlp=None),
])

# sizes that are no multiple of 8: a latent of 20, heads of 12 + 6, values of 10, a recurrence of 3 heads of 10, experts of 13
TAT_D = P.make_config(vocab=131, width=40, eps=1e-5, groups=5, mult=0.5, layers=[
    P.latent_layer(heads=3, dim=12, rot_dim=6, vdim=10, kv_rank=20, q_rank=12, window=None, rot_dims=4, base=20.0, mlp=P.experts_mlp(ff=13, experts=9, top=2, groups=(3, 2))),
    P.delta_layer(heads=3, dim=10, decay_rank=3, mlp=P.experts_mlp(ff=13, experts=5, top=2)),
    P.latent_layer(heads=2, dim=4, rot_dim=6, vdim=10, kv_rank=20, q_rank=9, window=5, rot_dims=4, base=20.0, kv_from=0, mlp=P.experts_mlp(ff=7, experts=3, top=3)),
])

TAT = {"A": (TAT_A, 11), "B": (TAT_B, 12), "C": (TAT_C, 13), "D": (TAT_D, 14)}
