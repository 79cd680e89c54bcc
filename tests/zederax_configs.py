"""Small Zederax configurations for the tests. They differ from layer to layer and from one another in every size and
option: heads equal to and a multiple of the key/value heads, one key/value head, key and value heads of equal and of
different size, windows shorter and longer than a page and none at all, layers without a soft cap, without a feed-forward
and without the value blend (also between two layers that have it)."""
import plain_zederax as Z

# windows 24 and 37 straddle pages of 16; the third layer sees every key; layer 2 does not blend, layers 1 and 3 do
ZED_A = Z.make_config(vocab=97, width=64, eps=1e-5, layers=[
    Z.layer(heads=4, kv_heads=2, dim=16, vdim=8, window=24, softcap=10.0, v_mix=True, ff=48),
    Z.layer(heads=4, kv_heads=2, dim=24, vdim=8, window=37, softcap=4.0, v_mix=False, ff=None),
    Z.layer(heads=2, kv_heads=2, dim=8, vdim=8, window=None, softcap=None, v_mix=True, ff=40),
    Z.layer(heads=6, kv_heads=1, dim=16, vdim=16, window=5, softcap=30.0, v_mix=False, ff=72),
])

# sizes the matrix-core kernels take (multiples of 16), one wide group, a window of exactly one page and one of one key
ZED_B = Z.make_config(vocab=211, width=96, eps=1e-6, layers=[
    Z.layer(heads=8, kv_heads=2, dim=32, vdim=16, window=16, softcap=15.0, v_mix=False, ff=112),
    Z.layer(heads=3, kv_heads=3, dim=16, vdim=32, window=70, softcap=8.0, v_mix=True, ff=64),
    Z.layer(heads=3, kv_heads=3, dim=48, vdim=32, window=1, softcap=None, v_mix=True, ff=None),
])

# one layer, one head: every list of the model has one entry
ZED_C = Z.make_config(vocab=50, width=32, eps=1e-3, layers=[
    Z.layer(heads=1, kv_heads=1, dim=8, vdim=24, window=9, softcap=2.0, v_mix=True, ff=16),
])

# head sizes that are no multiple of 8 (the engine stores such heads with zeros behind them), widths that are no multiple of 4
ZED_D = Z.make_config(vocab=61, width=50, eps=1e-5, layers=[
    Z.layer(heads=3, kv_heads=1, dim=12, vdim=20, window=19, softcap=6.0, v_mix=True, ff=30),
    Z.layer(heads=2, kv_heads=2, dim=20, vdim=10, window=None, softcap=None, v_mix=False, ff=33),
    Z.layer(heads=3, kv_heads=1, dim=36, vdim=20, window=50, softcap=12.0, v_mix=True, ff=None),
])

ZED = {"A": (ZED_A, 11), "B": (ZED_B, 12), "C": (ZED_C, 13), "D": (ZED_D, 14)}
