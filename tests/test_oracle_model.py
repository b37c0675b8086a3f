"""Pins the composition of the model oracle (oracle/niti_model_oracle.py) on the CPU: a training step of a
two-feature TiLinear, of a 1 x 1 TiConv2d and of a five-layer chain, worked out by hand from the reference's
statements (ti_torch.py:16-21 weight_update, 23-31 RoundShift, 48-69 PstoShift, 103-147 act_calc / err_calc /
grad_calc, 241-266 TiLinear, 268-290 TiReLU, 391-437 TiConv2d, 439-455 TiDropout, ti_net.py:17-32) and written
down as literals.  What these cases hold down: which exponent enters which sum (err_exp is advanced by
shift + weight_exp BEFORE weight_update reads it, a first layer never advances it), the operand order of the three
products, the shift of each rounding, both meanings of ``//`` and the pass-through layers' bookkeeping.

The arithmetic, for the pair of layers (they share every number: a 1 x 1 convolution over two pixels is the linear
layer over two samples):

  W = [[100, -50], [30, 127]] (out x in), weight_exp -7;  x = [[127, 64], [-104, 80]], exponent -3
  forward   x W^T = [[9500, 11938], [-14400, 7040]]; range 14400 -> 14 bits -> shift 7, exponent -3 - 7 + 7 = -3
            RoundShift(., 7): 9500 = 74*128 + 28 -> 74;  11938 = 93*128 + 34 -> 93;  7040 = 55*128 -> 55;
            -14400 = -(112*128 + 64), an exact tie: floor division gives -113*128 + 64 -> -113 + 1 = -112,
            truncating division gives -112*128 - 64 -> -112 - 1 = -113
  backward  err = [[5, -3], [-2, 7]], exponent -4
            err W = [[410, -631], [10, 989]]; range 989 -> 10 bits -> shift 3
            RoundShift(., 3): 410 = 51*8 + 2 -> 51;  -631 = -79*8 + 1 -> -79 (truncating: -78*8 - 7 -> -78 - 1);
            10 = 1*8 + 2 -> 1;  989 = 123*8 + 5 -> 124;  err_exp = -4 + 3 + (-7) = -8
            err^T x = [[843, 160], [-1109, 368]]; range 1109 -> 11 bits, mu 5 -> shift 6
            PstoShift(., 6) (remainder p, q = p // 8, r = p % 8, one more step away from zero when q > r):
            843 = 13*64 + 11: q 1, r 3 -> 13;  160 = 2*64 + 32: q 4, r 0 -> 3;  368 = 5*64 + 48: q 6, r 0 -> 6;
            -1109 floor: -18*64 + 43: q 5, r 3 -> -18 - 1 = -19;  truncating: -17*64 - 21: q 2, r 5 -> -17
            grad_exp = err_exp (-8, already advanced) + 6 + act_in_exp (-3) = -5; first layer: -4 + 6 - 3 = -1
            W - g = [[87, -53], [49, 121]] (floor) / [[87, -53], [47, 121]] (truncating)
"""
import pytest
import torch

from oracle import niti_model_oracle as mo

W = [[100, -50], [30, 127]]
X = [[127, 64], [-104, 80]]
ERR = [[5, -3], [-2, 7]]

EXPECT = {
    "floor": dict(y=[[74, 93], [-112, 55]], err_out=[[51, -79], [1, 124]], grad=[[13, 3], [-19, 6]],
                  w=[[87, -53], [49, 121]]),
    "trunc": dict(y=[[74, 93], [-113, 55]], err_out=[[51, -79], [1, 124]], grad=[[13, 3], [-17, 6]],
                  w=[[87, -53], [47, 121]]),
}


def i8(v):
    return torch.tensor(v, dtype=torch.int8)


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_linear_step_by_hand(div_mode):
    want = EXPECT[div_mode]
    cfg = mo.Cfg(div_mode=div_mode)
    lin = mo.OLinear(i8(W), -7)
    y, e = lin.forward((i8(X), -3), cfg)
    assert y.dtype == torch.int8 and y.tolist() == want["y"] and e == -3
    err_out, err_exp = lin.backward((i8(ERR), -4), cfg)
    assert err_out.tolist() == want["err_out"] and err_exp == -8 and lin.err_exp == -8
    assert lin.grad_int32acc.tolist() == [[843, 160], [-1109, 368]]
    assert lin.grad.tolist() == want["grad"] and lin.grad_shift == 6
    assert lin.grad_exp == -5
    assert lin.weight.tolist() == want["w"]


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
@pytest.mark.parametrize("first", [False, True])
def test_conv_1x1_step_by_hand(div_mode, first):
    """One image of 1 x 2 pixels, two channels in and out, 1 x 1 filter without padding: the two pixels are the
    linear layer's two samples.  A first layer returns None, leaves err_exp as it came in and takes its weight
    gradient through the grouped-convolution rewrite (ti_torch.py:194-233, 412-418)."""
    want = EXPECT[div_mode]
    cfg = mo.Cfg(div_mode=div_mode)
    conv = mo.OConv2d(i8(W).reshape(2, 1, 1, 2), -7, stride=1, padding=0, first_layer=first)
    y, e = conv.forward((i8(X).reshape(1, 1, 2, 2), -3), cfg)
    assert y.reshape(2, 2).tolist() == want["y"] and e == -3
    r = conv.backward((i8(ERR).reshape(1, 1, 2, 2), -4), cfg)
    assert conv.grad_int32acc.reshape(2, 2).tolist() == [[843, 160], [-1109, 368]]
    assert conv.grad.reshape(2, 2).tolist() == want["grad"] and conv.grad_shift == 6
    assert conv.weight.reshape(2, 2).tolist() == want["w"]
    if first:
        assert r is None
        assert conv.err_exp == -4 and conv.grad_exp == -1
    else:
        assert r[0].reshape(2, 2).tolist() == want["err_out"] and r[1] == -8
        assert conv.err_exp == -8 and conv.grad_exp == -5


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_chain_step_by_hand(div_mode):
    """conv 1 x 1 (first layer) -> ReLU -> Flat -> Dropout (mask [1, 0]) -> Linear, two images of one pixel.

    forward   conv as above: y = [[74, 93], [-112 | -113, 55]], exponent -3; ReLU: [[74, 93], [0, 55]];
              dropout: [[74, 0], [0, 0]], exponent -3 + 1 = -2
              linear W2 = [[3, 9], [-2, 5]], weight_exp -6: a W2^T = [[222, -148], [0, 0]]; range 222 -> 8 bits ->
              shift 1: [[111, -74], [0, 0]], exponent -2 - 6 + 1 = -7
    backward  err = [[4, -6], [8, 2]], exponent 0
              linear: err W2 = [[24, 6], [20, 82]]; range 82 -> 7 bits -> no shift, err_exp = 0 + 0 - 6 = -6
              err^T a = [[296, 0], [-444, 0]]; range 444 -> 9 bits, mu 5 -> shift 4; PstoShift(., 4) (q = p // 4,
              r = p % 4): 296 = 18*16 + 8: q 2, r 0 -> 19;  -444 floor: -28*16 + 4: q 1, r 0 -> -29;  truncating:
              -27*16 - 12: q 3, r 0 -> -28;  grad_exp = -6 + 4 + (-2) = -4;  W2 - g = [[-16, 9], [27 | 26, 5]]
              dropout: [[24, 0], [20, 0]]; ReLU (conv output > 0): [[24, 0], [0, 0]], exponent -6
              conv, first layer: err^T x = [[3048, 1536], [0, 0]]; range 3048 -> 12 bits -> shift 7;
              PstoShift(., 7) (q = p // 8, r = 2 (p % 8)): 3048 = 23*128 + 104: q 13, r 0 -> 24;  1536 = 12*128 -> 12
              grad_exp = -6 + 7 + (-3) = -2;  W - g = [[76, -62], [30, 127]];  returns None"""
    cfg = mo.Cfg(div_mode=div_mode)
    conv = mo.OConv2d(i8(W).reshape(2, 1, 1, 2), -7, stride=1, padding=0, first_layer=True)
    lin = mo.OLinear(i8([[3, 9], [-2, 5]]), -6)
    net = mo.ONet([conv, mo.OReLU(), mo.OFlat(), mo.ODropout(i8([1, 0])), lin], cfg)
    out, e = net.forward_int8(i8(X).reshape(2, 1, 1, 2), -3)
    assert out.tolist() == [[111, -74], [0, 0]] and e == -7
    assert [t[1] for t in net.trace] == [-3, -3, -3, -2, -7]
    r = net.backward_from(i8([[4, -6], [8, 2]]), 0)
    assert r is None
    assert lin.grad.tolist() == [[19, 0], [-29 if div_mode == "floor" else -28, 0]]
    assert lin.err_exp == -6 and lin.grad_shift == 4 and lin.grad_exp == -4
    assert lin.weight.tolist() == [[-16, 9], [27 if div_mode == "floor" else 26, 5]]
    # what the linear layer, the dropout and the ReLU hand down
    assert net.btrace[0][0].tolist() == [[24, 6], [20, 82]] and net.btrace[0][1] == -6
    assert net.btrace[1][0].tolist() == [[24, 0], [20, 0]] and net.btrace[1][1] == -6
    assert net.btrace[3][0].reshape(2, 2).tolist() == [[24, 0], [0, 0]] and net.btrace[3][1] == -6
    assert conv.grad_int32acc.reshape(2, 2).tolist() == [[3048, 1536], [0, 0]]
    assert conv.grad.reshape(2, 2).tolist() == [[24, 12], [0, 0]] and conv.grad_shift == 7
    assert conv.err_exp == -6 and conv.grad_exp == -2
    assert conv.weight.reshape(2, 2).tolist() == [[76, -62], [30, 127]]


def test_evaluation_mode_dropout_is_the_identity():
    """ti_torch.py:443-450: without TRAINING the dropout layer hands its input through, exponent included."""
    cfg = mo.Cfg(training=False)
    d = mo.ODropout(i8([1, 0]))
    a, e = d.forward((i8([[5, 6]]), -2), cfg)
    assert a.tolist() == [[5, 6]] and e == -2
