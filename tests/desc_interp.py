"""Test-only numpy interpreter of a dispatch descriptor.

It executes the kernel records of a descriptor the way the GPU kernels are
specified to (packed weights, split bias/scale, k-table gather, NHWC buffers,
transposes), so that the emitter's packing and layout decisions can be checked
against the oracle on a machine without a GPU.  It is not part of the product.
"""
import numpy as np

from oracle import oracle as orc

REF = np.dtype([("space", "<u4"), ("index", "<u4"), ("offset", "<u8")])
HEADER = np.dtype([("magic", "<u4"), ("version", "<u4"), ("arch", "<u4"), ("flags", "<u4"),
                   ("op_count", "<u4"), ("binding_count", "<u4"), ("temp_count", "<u4"), ("const_count", "<u4"),
                   ("ops_offset", "<u8"), ("bindings_offset", "<u8"), ("temps_offset", "<u8"),
                   ("consts_offset", "<u8"), ("data_offset", "<u8"), ("total_size", "<u8"), ("name", "S64")])
_I32 = ["out_dtype", "input_zp", "output_zp", "output_min", "output_max", "shift",
        "N", "H", "W", "C", "OH", "OW", "OC", "KH", "KW", "SH", "SW", "PL", "PR", "PT", "PB",
        "M", "K", "Kp", "Nn", "Np", "w0", "w1", "bias0", "scale0", "TB", "TR", "TS", "pre_shift", "t0_clamp", "TP"]
OP = np.dtype([("kind", "<u4"), ("variant", "<u4"), ("loader", "<u4"), ("gran", "<u4")] +
              [(n, "<i4") for n in _I32] +
              [(n, REF) for n in ["in0", "in1", "weights", "bias", "scale", "table", "out"]])
BINDING = np.dtype([("id", "<u4"), ("flags", "<u4"), ("size", "<u8")])
TEMP = np.dtype([("size", "<u8")])
CONST = np.dtype([("offset", "<u8"), ("size", "<u8")])

K_TRANSPOSE, K_IGEMM, K_FC_SKINNY, K_DW, K_MAXPOOL, K_AVGPOOL, K_ADD, K_FC_BF16, K_ADD_BF16, K_IM2COL_BF16, K_DW_BF16 = 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11
K_AVGPOOL_BF16, K_EXPAND, K_ELTWISE, K_DEC_LINEAR, K_DEC_MATMUL = 12, 13, 14, 15, 16
DEC_EXT = np.dtype([(n, REF, (3,)) for n in ["weights", "bias", "out"]] + [("N", "<i4", (3,)), ("has_qbias", "<i4"), ("res", REF), ("add_out", REF)] +
                   [(n, "<i4") for n in ["aw0", "aw1", "abias", "alo", "ahi"]] + [("reserved1", "<i4", (3,))])
INT_BY_SIZE = {1: np.int8, 2: np.int16, 4: np.int32}
OUT_NP = {1: np.int8, 2: np.int16, 3: np.int32}


class Descriptor:
    def __init__(self, blob):
        self.blob = np.frombuffer(blob, dtype=np.uint8)
        self.header = np.frombuffer(blob, dtype=HEADER, count=1)[0]
        h = self.header
        assert h["magic"] == 0x50494854 and h["total_size"] == len(blob)
        self.ops = np.frombuffer(blob, dtype=OP, count=int(h["op_count"]), offset=int(h["ops_offset"]))
        self.bindings = np.frombuffer(blob, dtype=BINDING, count=int(h["binding_count"]), offset=int(h["bindings_offset"]))
        self.temps = np.frombuffer(blob, dtype=TEMP, count=int(h["temp_count"]), offset=int(h["temps_offset"]))
        self.consts = np.frombuffer(blob, dtype=CONST, count=int(h["const_count"]), offset=int(h["consts_offset"]))

    def const_bytes(self, index):
        c = self.consts[index]
        start = int(self.header["data_offset"] + c["offset"])
        return self.blob[start:start + int(c["size"])]


_TYPE_RANGE = {np.int8: (-128, 127), np.int16: (-32768, 32767), np.int32: (-2 ** 31, 2 ** 31 - 1)}


def _requant_vec(acc, bias, scale, shift, zp, mn, mx, pre=0, t0_clamp=0):
    t0 = (acc.astype(np.int64) + bias.astype(np.int64))
    t0 = ((t0 + (1 << 31)) % (1 << 32)) - (1 << 31)  # int32 wrap
    if t0_clamp:
        assert pre and t0_clamp < (1 << (31 - pre))
        t0 = np.clip(t0, -t0_clamp, t0_clamp)
    if pre:
        # the kernels' 32-bit tail: (mulhi(t0 << pre, scale) + 1) >> 1, valid only if the shift loses no bit
        assert shift + pre == 33 and np.all(np.abs(t0) < (1 << (31 - pre))), "pre_shift overflows acc + bias"
        hi = ((t0 << pre) * scale.astype(np.int64)) >> 32
        return np.clip(((hi + 1) >> 1) + zp, mn, mx)
    t1 = t0 * scale.astype(np.int64)
    if shift > 0:
        t1 = t1 + (1 << (shift - 1))
    t3 = t1 >> shift
    return np.clip(t3 + zp, mn, mx)


def run(blob, binding_arrays):
    """Executes the descriptor on numpy arrays (one per binding, modified in place for outputs)."""
    d = Descriptor(blob)
    bufs = {1: [a.reshape(-1).view(np.uint8) for a in binding_arrays],
            2: [np.zeros(int(t["size"]), dtype=np.uint8) for t in d.temps],
            3: [d.const_bytes(i) for i in range(len(d.consts))]}

    def view(ref, nbytes):
        b = bufs[int(ref["space"])][int(ref["index"])]
        off = int(ref["offset"])
        assert off + nbytes <= b.size, "operand runs past its buffer"
        return b[off:off + nbytes]

    for op in d.ops:
        kind = int(op["kind"])
        sh, zp, mn, mx = int(op["shift"]), int(op["output_zp"]), int(op["output_min"]), int(op["output_max"])
        if kind == K_TRANSPOSE:
            B, R, S = int(op["TB"]), int(op["TR"]), int(op["TS"])
            pitch = int(op["TP"]) or R  # output rows `pitch` elements apart; what lies beyond R is left alone
            assert pitch >= R
            if int(op["gran"]) == 2:
                src = view(op["in0"], B * R * S * 2).view(np.uint16).reshape(B, R, S)
                view(op["out"], B * S * pitch * 2).view(np.uint16).reshape(B, S, pitch)[:, :, :R] = src.transpose(0, 2, 1)
                continue
            src = view(op["in0"], B * R * S).reshape(B, R, S)
            view(op["out"], B * S * pitch).reshape(B, S, pitch)[:, :, :R] = src.transpose(0, 2, 1)
        elif kind in (K_IGEMM, K_FC_SKINNY):
            M, K, Kp, N, Np = (int(op[k]) for k in ["M", "K", "Kp", "Nn", "Np"])
            Wp = view(op["weights"], Np * Kp).view(np.int8).reshape(Np, Kp).astype(np.int64)
            bias = view(op["bias"], Np * 4).view(np.int32)
            scale = view(op["scale"], Np * 4).view(np.int32)
            if kind == K_FC_SKINNY or int(op["loader"]) == 0:
                A = np.zeros((M, Kp), dtype=np.int64)
                A[:, :K] = view(op["in0"], M * K).view(np.int8).reshape(M, K)
            elif int(op["loader"]) == 2:  # one 16-byte run per window row: [kw][ci] bytes, zero-weight padding
                Nimg, H, W, C = (int(op[k]) for k in ["N", "H", "W", "C"])
                OH, OW, SH, SW, PT, PL = (int(op[k]) for k in ["OH", "OW", "SH", "SW", "PT", "PL"])
                x = view(op["in0"], Nimg * H * W * C).view(np.int8).reshape(Nimg, H, W, C)
                tab = view(op["table"], Kp // 16 * 4).view(np.uint32)
                A = np.zeros((Nimg, OH, OW, Kp), dtype=np.int64)
                oy = np.arange(OH)[:, None] * SH - PT
                ox = np.arange(OW)[None, :] * SW - PL
                for e, ent in enumerate(tab):
                    ent = int(ent)
                    if ent & 0x80000000:
                        continue
                    kh, length = (ent >> 24) & 0x7f, ent & 0xffff
                    assert length == int(op["KW"]) * C
                    for b in range(length):
                        kw, ci = b // C, b % C
                        iy, ix = oy + kh, ox + kw
                        inside = (iy >= 0) & (iy < H) & (ix >= 0) & (ix < W)
                        vals = x[:, np.clip(iy, 0, H - 1), np.clip(ix, 0, W - 1), ci].astype(np.int64)
                        A[..., e * 16 + b] = np.where(inside[None], vals, int(op["input_zp"]))
                    # bytes beyond the run are whatever memory holds: they must meet zero weights
                    A[..., e * 16 + length:(e + 1) * 16] = 77
                A = A.reshape(M, Kp)
            elif int(op["loader"]) == 3:  # the ring kernel's own window addressing: 16-byte chunk e holds channels (16 e) % C .. of tap 16 e // C
                Nimg, H, W, C = (int(op[k]) for k in ["N", "H", "W", "C"])
                OH, OW, SH, SW, PT, PL, KH, KW = (int(op[k]) for k in ["OH", "OW", "SH", "SW", "PT", "PL", "KH", "KW"])
                bk = 128 if int(op["variant"]) == 14 else 64
                assert int(op["variant"]) in (4, 5, 6, 7, 8, 9, 10, 14)
                assert C % 16 == 0 and K == KH * KW * C and Kp == -(-K // bk) * bk
                page = view(op["table"], 128).view(np.int8)
                assert (page == int(op["input_zp"])).all()
                x = view(op["in0"], Nimg * H * W * C).view(np.int8).reshape(Nimg, H, W, C)
                A = np.zeros((Nimg, OH, OW, Kp), dtype=np.int64)
                oy = np.arange(OH)[:, None] * SH - PT
                ox = np.arange(OW)[None, :] * SW - PL
                for e in range(Kp // 16):
                    tap, ci = (e * 16) // C, (e * 16) % C
                    if tap >= KH * KW:
                        # chunks of the last k-tile beyond K are whatever the walk reads: they must meet zero weights
                        A[..., e * 16:(e + 1) * 16] = 77
                        continue
                    kh, kw = tap // KW, tap % KW
                    iy, ix = oy + kh, ox + kw
                    inside = (iy >= 0) & (iy < H) & (ix >= 0) & (ix < W)
                    vals = x[:, np.clip(iy, 0, H - 1), np.clip(ix, 0, W - 1), ci:ci + 16].astype(np.int64)
                    A[..., e * 16:(e + 1) * 16] = np.where(inside[None, :, :, None], vals, int(page[0]))
                A = A.reshape(M, Kp)
            else:
                Nimg, H, W, C = (int(op[k]) for k in ["N", "H", "W", "C"])
                OH, OW, SH, SW, PT, PL = (int(op[k]) for k in ["OH", "OW", "SH", "SW", "PT", "PL"])
                g = int(op["gran"])
                x = view(op["in0"], Nimg * H * W * C).view(np.int8).reshape(Nimg, H, W, C)
                tab = view(op["table"], Kp // g * 4).view(np.uint32)
                A = np.zeros((Nimg, OH, OW, Kp), dtype=np.int64)
                oy = np.arange(OH)[:, None] * SH - PT
                ox = np.arange(OW)[None, :] * SW - PL
                for e, ent in enumerate(tab):
                    ent = int(ent)
                    if ent & 0x80000000:
                        continue
                    kh, kw, ci = (ent >> 24) & 0x7f, (ent >> 16) & 0xff, ent & 0xffff
                    iy, ix = oy + kh, ox + kw
                    inside = (iy >= 0) & (iy < H) & (ix >= 0) & (ix < W)
                    iyc, ixc = np.clip(iy, 0, H - 1), np.clip(ix, 0, W - 1)
                    vals = x[:, iyc, ixc, ci:ci + g].astype(np.int64)  # N,OH,OW,g
                    vals = np.where(inside[None, :, :, None], vals, int(op["input_zp"]))
                    A[..., e * g:(e + 1) * g] = vals
                A = A.reshape(M, Kp)
            # M x Np; as float64 through BLAS where that is exact (|acc| <= Kp * 2^14 < 2^53 always holds for int8 operands)
            assert Kp < (1 << 38)
            acc = np.rint(A.astype(np.float64) @ Wp.T.astype(np.float64)).astype(np.int64)
            q = _requant_vec(acc[:, :N], bias[None, :N], scale[None, :N], sh, zp, mn, mx, int(op["pre_shift"]), int(op["t0_clamp"]))
            odt = OUT_NP[int(op["out_dtype"])]
            res = q.astype(odt).reshape(-1)
            if kind == K_IGEMM and int(op["in1"]["space"]) != 0:
                # a residual add folded into the epilogue: the other operand from in1, the add's parameters from `table`
                assert int(op["variant"]) in (7, 11) and int(op["loader"]) == 0 and odt == np.int8
                ap = view(op["table"], 48).view(np.int32)
                other = view(op["in1"], M * N).view(np.int8)
                a, b = (other, res) if int(ap[8]) else (res, other)
                res = orc.add(a, b, np.array([ap[0], ap[1]], dtype=np.int16), np.array([ap[2], ap[3]], dtype=np.int32), output_zp=int(ap[5]),
                              output_min=int(ap[6]), output_max=int(ap[7]), shift_factor=int(ap[4]))
            out = view(op["out"], M * N * np.dtype(odt).itemsize).view(odt)
            out[:] = res
        elif kind == K_DW:
            Nimg, H, W, C, OH, OW = (int(op[k]) for k in ["N", "H", "W", "C", "OH", "OW"])
            KH, KW = int(op["KH"]), int(op["KW"])
            x = view(op["in0"], Nimg * H * W * C).view(np.int8).reshape(Nimg, H, W, C)
            if int(op["variant"]) == 1:  # [KH][C] dwords, byte kw = tap kw
                wd = view(op["weights"], KH * C * 4).view(np.int8).reshape(KH, C, 4)
                assert not wd[:, :, KW:].any()
                wpk = np.ascontiguousarray(wd[:, :, :KW].transpose(0, 2, 1))
            else:
                wpk = view(op["weights"], KH * KW * C).view(np.int8).reshape(KH, KW, C)
            sb = np.empty(2 * C, dtype=np.int32)
            sb[0::2] = view(op["bias"], C * 4).view(np.int32)
            sb[1::2] = view(op["scale"], C * 4).view(np.int32)
            w = np.ascontiguousarray(wpk.transpose(2, 0, 1))[:, None]
            res = orc.depthwise_conv2d(x, w, sb, input_zp=int(op["input_zp"]), output_zp=zp, output_min=mn,
                                       output_max=mx, shift_factor=sh,
                                       pad=[int(op["PL"]), int(op["PR"]), int(op["PT"]), int(op["PB"])],
                                       stride=[int(op["SH"]), int(op["SW"])], layout=orc.NHWC)
            assert res.shape == (Nimg, OH, OW, C)
            if int(op["pre_shift"]) and not int(op["t0_clamp"]):
                bound = 128 * np.abs(wpk.astype(np.int64)).sum(axis=(0, 1)) + np.abs(sb[0::2].astype(np.int64))
                assert sh + int(op["pre_shift"]) == 33 and np.all(bound < (1 << (31 - int(op["pre_shift"]))))
            view(op["out"], res.size)[:] = res.reshape(-1).view(np.uint8)
        elif kind == K_MAXPOOL:
            Nimg, H, W, C, OH, OW = (int(op[k]) for k in ["N", "H", "W", "C", "OH", "OW"])
            x = view(op["in0"], Nimg * H * W * C).view(np.int8).reshape(Nimg, H, W, C)
            res = orc.maxpool2d(x, input_zp=int(op["input_zp"]), output_min=mn, output_max=mx,
                                stride=[int(op["SH"]), int(op["SW"])],
                                pad=[int(op["PL"]), int(op["PR"]), int(op["PT"]), int(op["PB"])],
                                kernel=[int(op["KH"]), int(op["KW"])], layout=orc.NHWC)
            assert res.shape == (Nimg, OH, OW, C)
            view(op["out"], res.size)[:] = res.reshape(-1).view(np.uint8)
        elif kind == K_AVGPOOL:
            Nimg, H, W, C = (int(op[k]) for k in ["N", "H", "W", "C"])
            x = view(op["in0"], Nimg * H * W * C).view(np.int8).reshape(Nimg, H, W, C)
            res = orc.avg_pool2d(x, np.array([op["bias0"], op["scale0"]], dtype=np.int32), output_zp=zp,
                                 output_min=mn, output_max=mx, shift_factor=sh, weight=int(op["w0"]))
            view(op["out"], res.size)[:] = res.reshape(-1).view(np.uint8)
        elif kind == K_ADD:
            n = int(op["C"])
            a = view(op["in0"], n).view(np.int8)
            b = view(op["in1"], n).view(np.int8)
            res = orc.add(a, b, np.array([op["w0"], op["w1"]], dtype=np.int16),
                          np.array([op["bias0"], op["scale0"]], dtype=np.int32), output_zp=zp, output_min=mn,
                          output_max=mx, shift_factor=sh)
            view(op["out"], n)[:] = res.view(np.uint8)
        elif kind == K_IM2COL_BF16:
            Nimg, H, W, C, OH, OW, KH, KW = (int(op[k]) for k in ["N", "H", "W", "C", "OH", "OW", "KH", "KW"])
            SH, SW, PT, PL, Kp = (int(op[k]) for k in ["SH", "SW", "PT", "PL", "Kp"])
            x = view(op["in0"], Nimg * H * W * C * 2).view(np.uint16).reshape(Nimg, H, W, C)
            A = np.zeros((Nimg, OH, OW, Kp), dtype=np.uint16)
            oy = np.arange(OH)[:, None] * SH - PT
            ox = np.arange(OW)[None, :] * SW - PL
            for kh in range(KH):
                for kw in range(KW):
                    iy, ix = oy + kh, ox + kw
                    inside = (iy >= 0) & (iy < H) & (ix >= 0) & (ix < W)
                    vals = x[:, np.clip(iy, 0, H - 1), np.clip(ix, 0, W - 1), :]
                    k0 = (kh * KW + kw) * C
                    A[..., k0:k0 + C] = np.where(inside[None, :, :, None], vals, 0)
            view(op["out"], A.size * 2).view(np.uint16)[:] = A.reshape(-1)
        elif kind == K_DW_BF16:
            Nimg, H, W, C, OH, OW, KH, KW = (int(op[k]) for k in ["N", "H", "W", "C", "OH", "OW", "KH", "KW"])
            x = view(op["in0"], Nimg * H * W * C * 2).view(np.uint16).reshape(Nimg, H, W, C)
            wpk = view(op["weights"], KH * KW * C * 2).view(np.uint16).reshape(KH, KW, C)
            bias = view(op["bias"], C * 4).view(np.float32)
            res = orc.depthwise_conv2d_bf16(x, np.ascontiguousarray(wpk.transpose(2, 0, 1))[:, None], bias,
                                            pad=[int(op["PL"]), int(op["PR"]), int(op["PT"]), int(op["PB"])],
                                            stride=[int(op["SH"]), int(op["SW"])], output_min=mn, output_max=mx, layout=orc.NHWC)
            assert res.shape == (Nimg, OH, OW, C)
            view(op["out"], res.size * 2).view(np.uint16)[:] = res.reshape(-1)
        elif kind == K_ADD_BF16:
            n = int(op["C"])
            a = view(op["in0"], 2 * n).view(np.uint16)
            b = view(op["in1"], 2 * n).view(np.uint16)
            res = orc.add_bf16(a, b, np.array([op["w0"], op["w1"]], dtype=np.uint16),
                               np.array([op["bias0"]], dtype=np.int32).view(np.float32), output_min=mn, output_max=mx)
            view(op["out"], 2 * n).view(np.uint16)[:] = res
        elif kind == K_FC_BF16:
            M, K, N = int(op["M"]), int(op["K"]), int(op["Nn"])
            x = view(op["in0"], M * K * 2).view(np.uint16).reshape(M, K)
            if int(op["loader"]) == 2:  # block-quantized int8: [column block][k step][half][lane] x 16 bytes, tables [G][Np]
                steps, nbk = (K + 63) // 64, (N + 31) // 32
                block, cols = int(op["gran"]), int(op["Np"])
                G = K // block
                frag = view(op["weights"], nbk * 32 * steps * 64).view(np.int8).reshape(nbk, steps, 2, 2, 32, 16)  # [nb][s][h2][h][r][e]
                full = frag.transpose(0, 4, 1, 3, 2, 5).reshape(nbk * 32, steps * 64)  # [nb, r][s, h, h2, e]
                assert not full[N:].any() and not full[:, K:].any()
                sc = view(op["scale"], G * cols * 2).view(np.uint16).reshape(G, cols)
                bi = view(op["table"], G * cols * 4).view(np.float32).reshape(G, cols)
                wt = np.ascontiguousarray(orc.expand_weights(np.ascontiguousarray(full[:N, :K].T), sc[:, :N], bi, block_size=block,
                                                             output_min=int(op["bias0"]), output_max=int(op["scale0"])).T)
            elif int(op["loader"]) == 1:  # fragment order: [column block][k step][piece][lane] x 8 elements
                steps, nbk = (K + 63) // 64, (N + 31) // 32
                frag = view(op["weights"], nbk * 32 * steps * 64 * 2).view(np.uint16).reshape(nbk, steps, 4, 2, 32, 8)
                full = frag.transpose(0, 4, 1, 3, 2, 5).reshape(nbk * 32, steps * 64)  # [nb, r][s, h, c, e]
                assert not full[N:].any() and not full[:, K:].any()
                wt = np.ascontiguousarray(full[:N, :K])
            else:
                wt = view(op["weights"], N * K * 2).view(np.uint16).reshape(N, K)
            bias = view(op["bias"], N * 4).view(np.float32)
            res = orc.fully_connected_bf16(x, wt, bias, output_min=mn, output_max=mx)
            view(op["out"], M * N * 2).view(np.uint16)[:] = res.reshape(-1)
        elif kind == K_DEC_LINEAR:
            # grouped linear on block-quantized weights: every matrix as the expansion followed by the matmul, then the folded add
            M, K, block, nmat, flags = int(op["M"]), int(op["K"]), int(op["gran"]), int(op["w0"]), int(op["w1"])
            x = view(op["in0"], M * K * 2).view(np.uint16).reshape(M, K)
            ext = np.frombuffer(view(op["table"], DEC_EXT.itemsize).tobytes(), dtype=DEC_EXT, count=1)[0]
            G, kblocks = K // block, K // 128
            has_bias = int(ext["has_qbias"])
            slot = 2048 + 64 + (64 if has_bias else 0)
            ys = []
            for m in range(nmat):
                N = int(ext["N"][m])
                tiles = N // 16
                slots = view(ext["weights"][m], tiles * kblocks * slot).reshape(tiles, kblocks, slot)
                frag = np.ascontiguousarray(slots[:, :, :2048]).view(np.int8).reshape(tiles, kblocks, 2, 4, 16, 2, 8)  # [t][b][p][g][c][j & 1][e]
                full = frag.transpose(0, 4, 1, 2, 5, 3, 6).reshape(N, kblocks * 128)  # [t, c][b, p, j & 1, g, e]: k = 128 b + 32 (2 p + (j & 1)) + 8 g + e
                per_kb = np.ascontiguousarray(slots[:, :, 2048:2112]).view(np.float32).reshape(tiles, kblocks, 16).transpose(1, 0, 2).reshape(kblocks, N)
                assert np.array_equal(orc.from_bf16(orc.to_bf16(per_kb)), per_kb), "block scales are bf16 values"
                which = (np.arange(G) * block) // 128  # a quantisation block's scale is repeated in each of its k-blocks
                assert np.array_equal(per_kb, per_kb[which][(np.arange(kblocks) * 128) // block])
                sc = per_kb[which]
                bi = (np.ascontiguousarray(slots[:, :, 2112:2176]).view(np.float32).reshape(tiles, kblocks, 16).transpose(1, 0, 2).reshape(kblocks, N)[which]
                      if has_bias else np.zeros((G, N), np.float32))
                w16 = orc.expand_weights(np.ascontiguousarray(full.T), orc.to_bf16(sc), np.ascontiguousarray(bi), block_size=block,
                                         output_min=int(op["bias0"]), output_max=int(op["scale0"]))
                bias = view(ext["bias"][m], N * 4).view(np.float32)
                assert np.all(bias == bias[0])
                y = orc.matmul_bf16(x, w16, bias[:1], output_min=mn, output_max=mx)[0]
                ys.append(y)
                if int(ext["out"][m]["space"]):
                    view(ext["out"][m], M * N * 2).view(np.uint16)[:] = y.reshape(-1)
            if flags & 6:
                N = int(ext["N"][0])
                wts = np.array([ext["aw0"], ext["aw1"]], dtype=np.uint16)
                ab = np.array([ext["abias"]], dtype=np.int32).view(np.float32)
                if flags & 2:
                    res = view(ext["res"], M * N * 2).view(np.uint16).reshape(M, N).copy()
                    first, second = (res, ys[0]) if flags & 8 else (ys[0], res)
                else:
                    first, second = ys[0], ys[1]
                z = orc.add_bf16(first, second, wts, ab, output_min=int(ext["alo"]), output_max=int(ext["ahi"]))
                view(ext["add_out"], M * N * 2).view(np.uint16)[:] = z.reshape(-1)
        elif kind == K_DEC_MATMUL:
            B, M, K, N = int(op["TB"]), int(op["M"]), int(op["K"]), int(op["Nn"])
            a = view(op["in0"], (1 if int(op["w0"]) else B) * M * K * 2).view(np.uint16).reshape(-1, M, K)
            w = view(op["weights"], (1 if int(op["w1"]) else B) * N * K * 2).view(np.uint16).reshape(-1, N, K)
            res = orc.matmul_bf16(a, np.ascontiguousarray(w.transpose(0, 2, 1)), np.array([op["bias0"]], dtype=np.int32).view(np.float32),
                                  output_min=mn, output_max=mx)
            view(op["out"], B * M * N * 2).view(np.uint16)[:] = res.reshape(-1)
        elif kind == K_AVGPOOL_BF16:
            Nimg, H, W, C = (int(op[k]) for k in ["N", "H", "W", "C"])
            x = view(op["in0"], Nimg * H * W * C * 2).view(np.uint16).reshape(Nimg, H, W, C)
            res = orc.avg_pool2d_bf16(x, np.array([op["w0"]], dtype=np.uint16), np.array([op["bias0"]], dtype=np.int32).view(np.float32),
                                      output_min=mn, output_max=mx)
            view(op["out"], Nimg * C * 2).view(np.uint16)[:] = res.reshape(-1)
        elif kind == K_ELTWISE:
            n, variant, bcast = int(op["C"]), int(op["variant"]), int(op["w1"])
            tin, tout = INT_BY_SIZE[int(op["gran"])], OUT_NP[int(op["out_dtype"])]
            esz, osz = np.dtype(tin).itemsize, np.dtype(tout).itemsize
            a = view(op["in0"], (1 if bcast == 1 else n) * esz).view(tin)
            if variant == 0:
                res = orc.fma(a, [int(op["w0"])], [int(op["bias0"]), int(op["scale0"])], output_zp=zp, output_min=mn, output_max=mx,
                              shift_factor=sh, out_dtype=tout)
            elif variant == 1:
                b = view(op["in1"], (1 if bcast == 2 else n) * esz).view(tin)
                res = orc.mul(a, b, [int(op["bias0"]), int(op["scale0"])], output_zp=zp, output_min=mn, output_max=mx, shift=sh, out_dtype=tout)
            elif variant in (11, 18):  # bitwise / logical not
                assert tin == tout
                res = orc.elementwise_unary(3 if variant == 11 else 12, a.view(np.uint8) if variant == 18 else a)
                res = res.view(tout)
            elif 12 <= variant <= 17:  # comparisons and logical ops: a byte of 0 / 1 per element
                b = view(op["in1"], n * esz).view(tin)
                assert tout == np.int8
                if variant >= 15:
                    a, b = a.view(np.uint8), b.view(np.uint8)
                res = orc.elementwise_compare(variant - 6, a, b, is_unsigned=bool(int(op["w0"]))).view(np.int8)
            elif variant == 22:  # table: the record holds the 256 values in the output's type
                lut = view(op["in1"], 256 * osz).view(tout)
                assert osz >= esz and osz <= 2
                res = lut[(a.astype(np.int64) & 0xFF) ^ 0x80]
            elif variant >= 19:  # shifts
                b = view(op["in1"], n * esz).view(tin)
                assert tin == tout
                res = orc.elementwise_shift(variant - 19, a, b, round=bool(int(op["w0"])))
            elif variant >= 6:
                b = view(op["in1"], n * esz).view(tin)
                assert tin == tout
                res = orc.elementwise_binary({6: "and", 7: "or", 8: "xor", 9: "minimum", 10: "maximum"}[variant], a, b, is_unsigned=bool(int(op["w0"])))
            else:
                name = {2: "clamp", 3: "abs", 4: "negate", 5: "i2i"}[variant]
                if name != "clamp":  # the record carries the clip range the op implies
                    want = {"abs": _TYPE_RANGE[tout], "negate": _TYPE_RANGE[tout], "i2i": _TYPE_RANGE[np.int32]}[name]
                    assert (mn, mx) == want, (name, mn, mx)
                res = orc.act(a, name, min_int=mn, max_int=mx, out_dtype=tout)
            view(op["out"], n * osz).view(tout)[:] = res.reshape(-1)
        elif kind == K_EXPAND:
            K, N, block, cols = int(op["K"]), int(op["Nn"]), int(op["gran"]), int(op["Np"])
            G = K // block
            wq = view(op["in0"], K * N).view(np.int8).reshape(K, N)
            sc = view(op["scale"], G * N * 2).view(np.uint16).reshape(G, N)
            bi = view(op["bias"], G * cols * 4).view(np.float32).reshape(G, cols)
            res = orc.expand_weights(wq, sc, bi, block_size=block, output_min=mn, output_max=mx)
            view(op["out"], K * N * 2).view(np.uint16)[:] = res.reshape(-1)
        else:
            raise AssertionError("unknown kernel kind %d" % kind)
    return d
