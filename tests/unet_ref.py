"""The U-Net forward composed from oracle calls (checker of the whole-net parity tests): the same layer order, parameter order and
GroupNorm hand-offs as src/unet.c:588-607, :2567-2636, :2939-3105, every op evaluated by oracle/ on the host."""
import numpy as np

import orc


def dec_width(widths, dec_widths, i):
    """output channels of the block the decoder upsamples into level i - 1 (dw_of, src/unet.c:298-300): 0 or the bottom level: the encoder's"""
    return widths[i] if (i >= len(widths) - 1 or not dec_widths or i >= len(dec_widths) or not dec_widths[i]) else dec_widths[i]


def is_single(dec_convs, i):
    return bool(dec_convs) and i < len(dec_convs) and dec_convs[i] == 1


def param_layout(cin, widths, head_out, down_norm=0, dec_widths=None, dec_convs=None, enc_blocks=None, scale_cond=0):
    """dec_widths / dec_convs: cfg.dec_widths (a decoder block's width, 0 = the encoder's) and cfg.dec_convs (1: one conv, src/unet.c:357-362);
    enc_blocks: cfg.enc_blocks, residual blocks after encoder level i, their parameters after everything older (src/unet.c:461-465)"""
    L = len(widths); off = 0; lay = {}

    def conv(name, ci, co, k):
        nonlocal off
        lay[name + ".w"] = (off, (co, ci, k ** 3)); off += co * ci * k ** 3
        lay[name + ".b"] = (off, (co,)); off += co

    def gn(name, c):
        nonlocal off
        lay[name + ".gamma"] = (off, (c,)); off += c
        lay[name + ".beta"] = (off, (c,)); off += c

    for i in range(L):
        conv("enc%d.c1" % i, widths[i - 1] if i else cin, widths[i], 3); gn("enc%d.n1" % i, widths[i])
        conv("enc%d.c2" % i, widths[i], widths[i], 3); gn("enc%d.n2" % i, widths[i])
    for i in range(L - 1):
        conv("down%d" % i, widths[i], widths[i], 3)
    for i in range(L - 2, -1, -1):                   # the decoder blocks from the coarsest (src/unet.c:456)
        d = dec_width(widths, dec_widths, i)
        conv("dec%d.c1" % i, dec_width(widths, dec_widths, i + 1) + widths[i], d, 3); gn("dec%d.n1" % i, d)
        if not is_single(dec_convs, i):
            conv("dec%d.c2" % i, d, d, 3); gn("dec%d.n2" % i, d)
    conv("head", widths[0], head_out, 1)
    if down_norm:                                    # GroupNorm after each down conv, appended after the head (src/unet.c:459)
        for i in range(L - 1):
            gn("dn%d" % i, widths[i])
    if scale_cond:                                   # the voxel-size conditioning vector: widths[0] floats, before the residual blocks (src/unet.c:460)
        lay["scale_cond"] = (off, (widths[0],)); off += widths[0]
    for i, nb in enumerate(enc_blocks or []):
        for k in range(nb):
            conv("rb%d.%d.c1" % (i, k), widths[i], widths[i], 3); gn("rb%d.%d.n1" % (i, k), widths[i])
            conv("rb%d.%d.c2" % (i, k), widths[i], widths[i], 3); gn("rb%d.%d.n2" % (i, k), widths[i])
    return lay, off


def add_mx(bits, a, b, N, C, S):
    """y = a + b on MX tensors: decode, add in fp32, re-quantise (lp_add_mx, src/lp_mx_gn.cu:134-143)"""
    return orc.f32_to_mx(bits, orc.mx_to_f32(bits, a, N, C, S) + orc.mx_to_f32(bits, b, N, C, S), N, C, S)


def stored_stats(bits, y, N, c, g, S):
    sums = np.zeros((N, g, 2), np.float64)
    orc.lib().orc_gn_sums_mx(bits, orc.ptr(y), N, c, g, S, orc.ptr(sums), 0, S)
    mean = np.zeros(N * g, np.float32); rstd = np.zeros(N * g, np.float32)
    orc.lib().orc_gn_finalize(orc.ptr(sums), N * g, (c // g) * S, 1e-5, orc.ptr(mean), orc.ptr(rstd))
    return mean, rstd


def draw_order(lay):
    """The layout's keys with the decoder blocks from level 0 up (the encoder's order), wherever they sit in the flat vector: tests that draw
    random parameters key by key use it, so a seed names the same net whatever the flat layout is."""
    keys = list(lay)
    dec = [k for k in keys if k.startswith("dec")]
    if dec:
        first = keys.index(dec[0])
        keys[first:first + len(dec)] = sorted(dec, key=lambda k: (int(k[3:k.index(".")]), dec.index(k)))
    return keys


def slab_stats(bits, y, N, c, g, D, HW, zs):
    """cfg.l0_norm 4 (src/unet.c:992-1003): statistics [n][slab][G] of a stored level-0 tensor of at most 32 channels, slabs of zs planes: a pass
    over the tensor seen as n * slabs samples of zs planes (one channel block: a slab is a sample of the same layout)."""
    assert c <= 32 and D % zs == 0
    ns = D // zs
    sums = np.zeros((N * ns, g, 2), np.float64)
    orc.lib().orc_gn_sums_mx(bits, orc.ptr(y), N * ns, c, g, zs * HW, orc.ptr(sums), 0, zs * HW)
    mean = np.zeros(N * ns * g, np.float32); rstd = np.zeros(N * ns * g, np.float32)
    orc.lib().orc_gn_finalize(orc.ptr(sums), N * ns * g, (c // g) * zs * HW, 1e-5, orc.ptr(mean), orc.ptr(rstd))
    return mean, rstd


def forward(params, cin, widths, G, head_out, bits, xq, N, D, H, W, cbits=None, stored=0, down_norm=0, acc64=0, l0_slab=0, dec_widths=None, dec_convs=None, enc_blocks=None):
    """xq: MX bytes of the input. Returns (logits fp32 [N][head_out][S], {layer name: MX bytes}). acc64: the convs' contraction summed in
    double and rounded once (else in fp32, block by block): two correct summation orders of the same graph. l0_slab > 0: cfg.l0_norm 4, the
    level-0 GroupNorms on statistics per z-slab of that many planes."""
    lay, n = param_layout(cin, widths, head_out, down_norm, dec_widths, dec_convs, enc_blocks)
    assert params.size == n
    P = lambda k: np.ascontiguousarray(params[lay[k][0]:lay[k][0] + int(np.prod(lay[k][1]))].reshape(lay[k][1]))
    L = len(widths); dt = 3 if bits == 8 else 4
    outs = {}
    Gof = lambda c: min(G, c)
    dims = [(D >> i, H >> i, W >> i) for i in range(L)]

    live = []

    def l0gn(i, norm, y, ms, c=None):
        """the GroupNorm a reader of level i's tensor y (c channels) applies: per-sample statistics ms, or, at level 0 under l0_slab, the tensor's per-slab ones"""
        c = c or widths[i]; g = Gof(c)
        if i == 0 and l0_slab:
            m, r = slab_stats(bits, y, N, c, g, D, H * W, l0_slab)
            live.append((m, r))                  # (the descriptor holds plain addresses)
            return orc.gn(P(norm + ".gamma"), P(norm + ".beta"), m, r, g, slab=(l0_slab, 0, D // l0_slab, H * W)), (m, r)
        return orc.gn(P(norm + ".gamma"), P(norm + ".beta"), ms[0], ms[1], g), ms

    def finalize(sums, c, S):
        g = Gof(c)
        mean = np.zeros(N * g, np.float32); rstd = np.zeros(N * g, np.float32)
        orc.lib().orc_gn_finalize(orc.ptr(sums), N * g, (c // g) * S, 1e-5, orc.ptr(mean), orc.ptr(rstd))
        return mean, rstd

    def conv(name, x, ci, d, gp=None, x2=None, c_split=0, up=0, gp2=None, stride=1, stats=True):
        co = lay[name + ".w"][1][0]
        cb = cbits if (cbits and ci > 8) else (4 if (bits == 4 and ci > 8) else 8)
        if stride == 2:                       # the reference's stride-2 dispatch: fp4 only for an MX-fp4 32 -> <= 32 channel conv (src/lp_s2.cu:653-671)
            cb = 4 if (bits == 4 and ci == 32 and co <= 32) else 8
        y, s = orc.conv3(x, dt, N, ci, d[0], d[1], d[2], P(name + ".w"), P(name + ".b"), co, dt, cbits=cb, stride=stride, x2=x2, c_split=c_split, up=up,
                         gp=gp, gp2=gp2, Go=Gof(co), want_stats=stats, stored_stats=stored, acc64=acc64,
                         stem_tile=int(ci <= 8 and stride == 1 and x2 is None))   # the network input: tap-packed kernel, one scale per tile (src/lp_f8fwd.cuh:601-609)
        outs[name] = y
        return y, s

    cur, blocks, gin = xq, {}, None
    for i in range(L):
        ci = widths[i - 1] if i else cin
        S = dims[i][0] * dims[i][1] * dims[i][2]
        a1, s1 = conv("enc%d.c1" % i, cur, ci, dims[i], gp=gin)
        m1, r1 = finalize(s1, widths[i], S)
        a2, s2 = conv("enc%d.c2" % i, a1, widths[i], dims[i], gp=l0gn(i, "enc%d.n1" % i, a1, (m1, r1))[0])
        m2, r2 = finalize(s2, widths[i], S)
        g2, (m2, r2) = l0gn(i, "enc%d.n2" % i, a2, (m2, r2))
        blocks["enc%d" % i] = (a2, g2, (m2, r2))
        for k in range((enc_blocks or [0] * L)[i]):      # residual blocks (rblock_fwd, src/unet.c:2656-2671): the stage output replaces enc<i>'s
            nm = "rb%d.%d" % (i, k); prev = blocks["enc%d" % i]
            b1, t1 = conv(nm + ".c1", prev[0], widths[i], dims[i], gp=prev[1])
            bm1, br1 = finalize(t1, widths[i], S)
            b2, _ = conv(nm + ".c2", b1, widths[i], dims[i], gp=orc.gn(P(nm + ".n1.gamma"), P(nm + ".n1.beta"), bm1, br1, Gof(widths[i])), stats=False)
            b2 = add_mx(bits, b2, prev[0], N, widths[i], S); outs[nm + ".c2"] = b2
            bm2, br2 = stored_stats(bits, b2, N, widths[i], Gof(widths[i]), S)
            live.append((bm1, br1, bm2, br2))
            blocks["enc%d" % i] = (b2, orc.gn(P(nm + ".n2.gamma"), P(nm + ".n2.beta"), bm2, br2, Gof(widths[i])), (bm2, br2))
            a2 = b2
        if i < L - 1:
            cur, _ = conv("down%d" % i, a2, widths[i], dims[i], gp=blocks["enc%d" % i][1], stride=2, stats=False)
            if down_norm:                     # statistics of the stored down-conv output, applied by the next conv1 (src/unet.c:2974-2979)
                Sd = dims[i + 1][0] * dims[i + 1][1] * dims[i + 1][2]; g = Gof(widths[i])
                sums = np.zeros((N, g, 2), np.float64)
                orc.lib().orc_gn_sums_mx(bits, orc.ptr(cur), N, widths[i], g, Sd, orc.ptr(sums), 0, Sd)
                md, rd = finalize(sums, widths[i], Sd)
                gin = orc.gn(P("dn%d.gamma" % i), P("dn%d.beta" % i), md, rd, g)
    for i in range(L - 2, -1, -1):
        coarse = blocks["enc%d" % (L - 1)] if i == L - 2 else blocks["dec%d" % (i + 1)]
        skip = blocks["enc%d" % i]
        S = dims[i][0] * dims[i][1] * dims[i][2]
        dw, dc = dec_width(widths, dec_widths, i), dec_width(widths, dec_widths, i + 1)
        a1, s1 = conv("dec%d.c1" % i, coarse[0], dc + widths[i], dims[i], gp=coarse[1], x2=skip[0], c_split=dc, up=1, gp2=skip[1])
        m1, r1 = finalize(s1, dw, S)
        if is_single(dec_convs, i):                   # one conv: its output is the block's, under n1 (src/unet.c:2581-2582)
            g1, (m1, r1) = l0gn(i, "dec%d.n1" % i, a1, (m1, r1), dw)
            blocks["dec%d" % i] = (a1, g1, (m1, r1))
            continue
        a2, s2 = conv("dec%d.c2" % i, a1, dw, dims[i], gp=l0gn(i, "dec%d.n1" % i, a1, (m1, r1), dw)[0])
        m2, r2 = finalize(s2, dw, S)
        g2, (m2, r2) = l0gn(i, "dec%d.n2" % i, a2, (m2, r2), dw)
        blocks["dec%d" % i] = (a2, g2, (m2, r2))
    last = blocks["dec0"] if L > 1 else blocks["enc0"]
    S = D * H * W
    logits = np.zeros((N, head_out, S), np.float32)
    hw = np.ascontiguousarray(P("head.w").reshape(head_out, widths[0])); hb = P("head.b")
    orc.lib().orc_conv1_mx(bits, orc.ptr(last[0]), N, widths[0], S, orc.ptr(hw), orc.ptr(hb), head_out, last[1], orc.ptr(logits))
    return logits, outs


def layer_inputs(widths, dec_convs=None, enc_blocks=None):
    """name -> (x layer, x2 layer, stride, up) of every conv in execution order; 'input' is the network input. The GroupNorm a reader
    applies is the statistics of the tensor it reads with the parameters of the block norm that follows that tensor."""
    L = len(widths); g = []
    dout = lambda i: "dec%d.c%d" % (i, 1 if is_single(dec_convs, i) else 2)
    nrb = lambda i: (enc_blocks or [0] * L)[i] if i < len(enc_blocks or [0] * L) else 0
    eout = lambda i: "rb%d.%d.c2" % (i, nrb(i) - 1) if nrb(i) else "enc%d.c2" % i      # the stage output: the last residual block's (a rb c2 tensor is its conv + the previous output)
    for i in range(L):
        g.append(("enc%d.c1" % i, "input" if i == 0 else "down%d" % (i - 1), None, 1, 0))
        g.append(("enc%d.c2" % i, "enc%d.c1" % i, None, 1, 0))
        for k in range(nrb(i)):
            g.append(("rb%d.%d.c1" % (i, k), "rb%d.%d.c2" % (i, k - 1) if k else "enc%d.c2" % i, None, 1, 0))
            g.append(("rb%d.%d.c2" % (i, k), "rb%d.%d.c1" % (i, k), None, 1, 0))
        if i < L - 1:
            g.append(("down%d" % i, eout(i), None, 2, 0))
    for i in range(L - 2, -1, -1):
        coarse = eout(L - 1) if i == L - 2 else dout(i + 1)
        g.append(("dec%d.c1" % i, coarse, eout(i), 1, 1))
        if not is_single(dec_convs, i):
            g.append(("dec%d.c2" % i, "dec%d.c1" % i, None, 1, 0))
    return g


def norm_of(layer, down_norm=0):
    """the GroupNorm parameters applied to a conv output by its readers: block.c1 -> block.n1, block.c2 -> block.n2; down convs: none,
    or dn<i> with down_norm."""
    if layer.startswith("down"):
        return "dn" + layer[4:] if down_norm else None
    if layer == "input":
        return None
    blk, c = layer.rsplit(".", 1)
    return blk + (".n1" if c == "c1" else ".n2")
