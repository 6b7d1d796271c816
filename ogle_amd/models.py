"""Graph generators for the workloads the benchmarks and tests run.

No model file of the reference is available offline, so graphs are built in code
with seeded random weights, in the form the reference's converter would emit:
batch-norm and ReLU6 already folded into each convolution
(converter/converter/optimizers/remapper.cc:97-176), filters as OIHW constants.
"""
import numpy as np

from . import dlx


def fold_batchnorm(w, bias, gamma, beta, mean, var, eps=1e-5):
    """Conv -> BN folding, fp32 throughout (remapper.cc:142-149):
    scale = gamma / sqrt(var + eps); w[o] *= scale; b = b*scale + (beta - scale*mean).
    A conv without bias gets a zero bias first (remapper.cc:124-134)."""
    w = np.asarray(w, np.float32)
    o = w.shape[0]
    bias = np.zeros(o, np.float32) if bias is None else np.asarray(bias, np.float32)
    f32 = np.float32
    scale = (np.asarray(gamma, f32) / np.sqrt(np.asarray(var, f32) + f32(eps))).astype(f32)
    shift = (-scale * np.asarray(mean, f32) + np.asarray(beta, f32)).astype(f32)
    wf = (w.reshape(o, -1) * scale[:, None]).astype(f32).reshape(w.shape)
    bf = (bias * scale + shift).astype(f32)
    return wf, bf


def ssd_anchors(maps=(19, 10, 5, 3, 2, 1), counts=(3, 6, 6, 6, 6, 6), smin=0.2, smax=0.95):
    """Center-size priors (cx, cy, w, h): scales linear in [smin, smax] over the maps, aspect
    ratios {1, 2, 1/2} (+ {3, 1/3} and the extra sqrt(s_k s_k+1) box where a map has 6)."""
    k = len(maps)
    scales = [smin + (smax - smin) * i / (k - 1) for i in range(k)] + [1.0]
    out = []
    for i, (m, a) in enumerate(zip(maps, counts)):
        ratios = [1.0, 2.0, 0.5] if a == 3 else [1.0, 2.0, 0.5, 3.0, 1.0 / 3.0]
        for y in range(m):
            for x in range(m):
                cx, cy = (x + 0.5) / m, (y + 0.5) / m
                for ar in ratios:
                    out.append([cx, cy, scales[i] * np.sqrt(ar), scales[i] / np.sqrt(ar)])
                if a == 6:
                    s = np.sqrt(scales[i] * scales[i + 1])
                    out.append([cx, cy, s, s])
    return np.array(out, np.float32)


MOBILENET_V1_BLOCKS = [  # (out channels, stride of the depthwise conv)
    (64, 1), (128, 2), (128, 1), (256, 2), (256, 1), (512, 2), (512, 1), (512, 1), (512, 1),
    (512, 1), (512, 1), (1024, 2), (1024, 1)]
SSD_EXTRAS = [(256, 512), (128, 256), (128, 256), (64, 128)]  # (1x1 channels, 3x3-s2 channels)
SSD_ANCHORS_PER_MAP = (3, 6, 6, 6, 6, 6)


def mobilenet_v1_ssd(batch, seed=20240005, num_classes=21, image=300, head_std=0.01,
                     with_weights=False):
    """MobileNet-v1 SSD 300x300: 3x3-s2 stem, 13 depthwise-separable blocks (32 -> 1024),
    4 extra 1x1 / 3x3-s2 pairs, 6 loc + 6 conf 3x3 heads on the maps of block 11, block 13 and
    the extras, concatenated to box_preds (N, 1917, 4) and cls_logits (N, 1917, classes).
    BN (gamma~U(.5,1.5), beta, mean~N(0,.1), var~U(.5,1.5)) is folded; activation ReLU6 as
    Clip(0, 6).  Returns (GraphBuilder, info) where info lists every conv layer
    (name, kind, shapes) and, if with_weights, the folded weights for an oracle run plus, under
    "unfolded", what they were folded from: name -> (w, gamma, beta, mean, var), or (w,) for a
    head."""
    r = np.random.Generator(np.random.PCG64(seed))
    g = dlx.GraphBuilder()
    x = g.add_input("input", [batch, 3, image, image])
    layers = []
    weights = {}
    unfolded = {}

    def conv_bn(name, x, cin, cout, k, stride, pad, group=1, bn=True, act=True, std=None):
        fan_in = (cin // group) * k * k
        std = np.sqrt(2.0 / fan_in) if std is None else std
        w = r.normal(0, std, (cout, cin // group, k, k)).astype(np.float32)
        b = None
        if with_weights:
            unfolded[name] = (w,)
        if bn:
            gamma = r.uniform(0.5, 1.5, cout).astype(np.float32)
            beta = r.normal(0, 0.1, cout).astype(np.float32)
            mean = r.normal(0, 0.1, cout).astype(np.float32)
            var = r.uniform(0.5, 1.5, cout).astype(np.float32)
            if with_weights:
                unfolded[name] = (w, gamma, beta, mean, var)
            w, b = fold_batchnorm(w, None, gamma, beta, mean, var)
        wi = g.add_filter(name + ".weight", w)
        bi = g.add_const(name + ".bias", b) if b is not None else None
        y = g.add_conv(name, x, wi, bi, k, stride, pad, 1, group, "Clip" if act else "",
                       0.0, 6.0 if act else 0.0)
        kind = "dw" if group == cin and group > 1 else ("pw" if k == 1 else "dense")
        layers.append(dict(name=name, kind=kind, cin=cin, cout=cout, k=k, stride=stride, pad=pad,
                           group=group, act=act))
        if with_weights:
            weights[name] = (w, b)
        return y

    size = image
    x = conv_bn("conv0", x, 3, 32, 3, 2, 1)
    size = (size - 3 + 2) // 2 + 1
    layers[-1]["in_size"] = image
    c = 32
    feature_maps = []
    for i, (cout, stride) in enumerate(MOBILENET_V1_BLOCKS, start=1):
        layers_before = len(layers)
        x = conv_bn("block%d.dw" % i, x, c, c, 3, stride, 1, group=c)
        layers[layers_before]["in_size"] = size
        size = (size - 3 + 2) // stride + 1
        x = conv_bn("block%d.pw" % i, x, c, cout, 1, 1, 0)
        layers[-1]["in_size"] = size
        c = cout
        if i in (11, 13):
            feature_maps.append((x, c, size))
    for i, (c1, c2) in enumerate(SSD_EXTRAS, start=1):
        x = conv_bn("extra%d.pw" % i, x, c, c1, 1, 1, 0)
        layers[-1]["in_size"] = size
        x = conv_bn("extra%d.conv" % i, x, c1, c2, 3, 2, 1)
        layers[-1]["in_size"] = size
        size = (size - 3 + 2) // 2 + 1
        c = c2
        feature_maps.append((x, c, size))

    locs, confs = [], []
    priors = 0
    for i, ((fx, fc, fs), a) in enumerate(zip(feature_maps, SSD_ANCHORS_PER_MAP)):
        priors += fs * fs * a
        for kind, last, acc in (("loc", 4, locs), ("conf", num_classes, confs)):
            name = "head%d.%s" % (i, kind)
            y = conv_bn(name, fx, fc, a * last, 3, 1, 1, bn=False, act=False, std=head_std)
            layers[-1]["in_size"] = fs
            # PyTorch-style head: permute(0,2,3,1) then view(N,-1,last).  The ONNX perm is
            # over NCHW axes; on NHWC storage it is the identity.
            t = g.add_transpose(name + ".permute", y, [0, 2, 3, 1])
            shp = g.add_const(name + ".shape", np.array([batch, -1, last], np.float32))
            acc.append(g.add_reshape(name + ".view", t, shp))
    g.add_concat("box_preds", locs, 1)
    g.add_concat("cls_logits", confs, 1)
    anchors = ssd_anchors()
    assert anchors.shape[0] == priors
    g.add_const("anchors", anchors)
    for name in ("cls_logits", "box_preds", "anchors"):
        g.add_output_name(name)
    for l in layers:
        out_size = (l["in_size"] - l["k"] + 2 * l["pad"]) // l["stride"] + 1
        l["out_size"] = out_size
        macs = out_size * out_size * l["cout"] * (l["cin"] // l["group"]) * l["k"] ** 2
        l["flops_per_image"] = 2 * macs
        w_elems = l["cout"] * (l["cin"] // l["group"]) * l["k"] ** 2
        l["weight_bytes"] = 4 * (w_elems + (l["cout"] if l["name"].find("head") < 0 else 0))
        l["act_bytes_per_image"] = 4 * (l["in_size"] ** 2 * l["cin"] + out_size ** 2 * l["cout"])
    info = dict(layers=layers, priors=priors, num_classes=num_classes, weights=weights,
                unfolded=unfolded, anchors=anchors, seed=seed)
    return g, info


def separable_block(batch, seed=20240002, size=38, cin=256, cout=512):
    """BASELINE config 2: depthwise 3x3 s1 p1 + BN + ReLU6, pointwise 1x1 + BN + ReLU6."""
    r = np.random.Generator(np.random.PCG64(seed))
    g = dlx.GraphBuilder()
    x = g.add_input("input", [batch, cin, size, size])

    def bn(c):
        return (r.uniform(0.5, 1.5, c).astype(np.float32), r.normal(0, 0.1, c).astype(np.float32),
                r.normal(0, 0.1, c).astype(np.float32), r.uniform(0.5, 1.5, c).astype(np.float32))

    wd = r.normal(0, np.sqrt(2 / 9), (cin, 1, 3, 3)).astype(np.float32)
    wp = r.normal(0, np.sqrt(2 / cin), (cout, cin, 1, 1)).astype(np.float32)
    wd, bd = fold_batchnorm(wd, None, *bn(cin))
    wp, bp = fold_batchnorm(wp, None, *bn(cout))
    y = g.add_conv("dw", x, g.add_filter("dw.weight", wd), g.add_const("dw.bias", bd), 3, 1, 1, 1,
                   cin, "Clip", 0.0, 6.0)
    g.add_conv("pw", y, g.add_filter("pw.weight", wp), g.add_const("pw.bias", bp), 1, 1, 0, 1, 1,
               "Clip", 0.0, 6.0)
    g.add_output_name("pw")
    return g, dict(wd=wd, bd=bd, wp=wp, bp=bp)
