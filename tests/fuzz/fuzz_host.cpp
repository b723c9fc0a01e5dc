// Host-side fuzz of the emitter and the descriptor validation, meant to be built with
// -fsanitize=address,undefined (tests/test_fuzz.py does that and runs it).  Nothing here touches a GPU.
//
//   1. random programs through the C-ABI emitter (thip_program_* / thip_hl_*): single int8 ops and decode-shaped bf16
//      programs (grouped linears on block-quantized weights, views, folded transposes), sane and insane attribute
//      values; every call must come back with a status;
//   2. every blob the emitter produces must validate; mutated copies (bit flips in the header, the kernel records,
//      the tables; truncations) must come back with a status, never a crash or a sanitizer report;
//   3. the CPU oracle on small random shapes (its indexing under the address sanitizer).
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <vector>

#include "../../include/thip.h"
#include "../../oracle/torq_oracle.h"
#include "../../torq-compiler_amd/csrc/thip_descriptor.h"

static std::mt19937_64 rng(20261125);
static int64_t pick(int64_t lo, int64_t hi) { return lo + (int64_t)(rng() % (uint64_t)(hi - lo + 1)); }
static int32_t wild() {
    switch (rng() % 6) {
    case 0: return 0;
    case 1: return -1;
    case 2: return INT32_MAX;
    case 3: return INT32_MIN;
    case 4: return (int32_t)pick(-300, 300);
    default: return (int32_t)rng();
    }
}

struct Blob {
    std::vector<uint64_t> words;  // 8-byte aligned storage
    size_t size = 0;
    uint8_t *data() { return (uint8_t *)words.data(); }
};

static thip_value_t constantI8(thip_program_t *p, std::vector<int64_t> shape) {
    size_t n = 1;
    for (int64_t d : shape) n *= (size_t)d;
    std::vector<int8_t> v(n);
    for (auto &x : v) x = (int8_t)rng();
    thip_value_t id = -1;
    thip_program_constant(p, THIP_DTYPE_I8, (int32_t)shape.size(), shape.data(), v.data(), v.size(), &id);
    return id;
}
static thip_value_t constantI32(thip_program_t *p, size_t n) {
    std::vector<int32_t> v(n);
    for (auto &x : v) x = (int32_t)pick(1, 1 << 30);
    int64_t shape[1] = {(int64_t)n};
    thip_value_t id = -1;
    thip_program_constant(p, THIP_DTYPE_I32, 1, shape, v.data(), v.size() * 4, &id);
    return id;
}
static thip_value_t binding(thip_program_t *p, uint32_t index, std::vector<int64_t> shape, int32_t dtype = THIP_DTYPE_I8) {
    thip_value_t id = -1;
    thip_program_binding(p, index, dtype, (int32_t)shape.size(), shape.data(), &id);
    return id;
}

static thip_value_t constantRaw(thip_program_t *p, int32_t dtype, std::vector<int64_t> shape, size_t elemBytes, int fill) {
    size_t n = 1;
    for (int64_t d : shape) n *= (size_t)d;
    std::vector<uint8_t> v(n * elemBytes);
    for (auto &x : v) x = fill < 0 ? (uint8_t)rng() : (uint8_t)fill;
    if (dtype == THIP_DTYPE_BF16 && fill < 0) {
        for (size_t i = 0; i < n; i++) v[2 * i + 1] = (uint8_t)(0x3b + (rng() & 3));  // finite, small
    }
    thip_value_t id = -1;
    thip_program_constant(p, dtype, (int32_t)shape.size(), shape.data(), v.data(), v.size(), &id);
    return id;
}

// A decode-shaped bf16 program: one to three linears on block-quantized int8 weights over the same rows (sometimes a
// pair joined by an add, sometimes a residual add behind one), results into bindings, intermediates or views of a
// binding, and sometimes a small matmul against a transposed run-time operand -- the shapes the grouping and the
// slot packing of the serialiser are written for, and the ones just outside them.
static thip_status_t buildDecodeProgram(thip_program_t *p, bool insane) {
    const int64_t M = insane ? pick(1, 40) : pick(1, 32);
    const int64_t block = (rng() % 4 == 0) ? 64 * pick(1, 5) : 128 * pick(1, 2);
    const int64_t K = (rng() % 5 == 0) ? 16 * pick(1, 30) : block * pick(1, 4);
    const int32_t noLo = (int32_t)0xff800000, noHi = 0x7f800000;
    uint32_t nextBinding = 0;
    const thip_value_t x = binding(p, nextBinding++, {M, K}, THIP_DTYPE_BF16);
    const thip_value_t zero = constantRaw(p, THIP_DTYPE_F32, {1}, 4, 0);
    const int mode = (int)(rng() % 5);  // 0 single, 1 several on the same rows, 2 pair + add, 3 residual add, 4 attention-shaped matmul
    auto linear = [&](int64_t N, thip_value_t init, thip_value_t *result) -> thip_status_t {
        if (K % block != 0) return THIP_INVALID_ARGUMENT;  // no such expansion exists
        const int64_t G = K / block;
        thip_hl_expand_weights_t e;
        memset(&e, 0, sizeof(e));
        e.input = constantRaw(p, THIP_DTYPE_I8, {K, N}, 1, -1);
        e.scale = constantRaw(p, THIP_DTYPE_BF16, {G, N}, 2, -1);
        e.scale_bias = constantRaw(p, THIP_DTYPE_F32, {G, N + (N & 1)}, 4, (rng() & 1) ? 0 : 0x3c);
        e.block_size = insane && rng() % 4 == 0 ? wild() : (int32_t)block;
        e.output_min = noLo;
        e.output_max = noHi;
        int64_t wshape[2] = {K, N};
        if (thip_status_t s = thip_program_tensor(p, THIP_DTYPE_BF16, 2, wshape, &e.init)) return s;
        if (thip_status_t s = thip_hl_expand_weights(p, &e)) return s;
        thip_hl_matmul_t m;
        memset(&m, 0, sizeof(m));
        m.init = init;
        m.output_min = noLo;
        m.output_max = noHi;
        m.shift = insane && rng() % 6 == 0 ? wild() : 0;
        m.scale_bias = zero;
        m.input1 = x;
        m.input2 = e.init;
        *result = init;
        return thip_hl_matmul(p, &m);
    };
    auto result = [&](int64_t N, int how) -> thip_value_t {  // how: 0 binding, 1 intermediate, 2 a view into a larger binding
        thip_value_t v = -1;
        int64_t shape[2] = {M, N};
        if (how == 1) {
            thip_program_tensor(p, THIP_DTYPE_BF16, 2, shape, &v);
        } else if (how == 2) {
            const thip_value_t base = binding(p, nextBinding++, {3, M, N}, THIP_DTYPE_BF16);
            thip_program_view(p, base, (insane && rng() % 3 == 0 ? (int64_t)wild() : M * N * pick(0, 2)), 2, shape, &v);
        } else {
            v = binding(p, nextBinding++, {M, N}, THIP_DTYPE_BF16);
        }
        return v;
    };
    auto add = [&](thip_value_t a, thip_value_t b, int64_t N) -> thip_status_t {
        thip_hl_add_t c;
        memset(&c, 0, sizeof(c));
        c.init = binding(p, nextBinding++, {M, N}, THIP_DTYPE_BF16);
        c.output_min = noLo;
        c.output_max = noHi;
        c.weights = constantRaw(p, THIP_DTYPE_BF16, {2}, 2, -1);
        c.scale_bias = constantRaw(p, THIP_DTYPE_F32, {1}, 4, 0);
        c.input1 = a;
        c.input2 = b;
        return thip_hl_add(p, &c);
    };
    const int64_t N = (rng() % 5 == 0) ? pick(1, 70) : 16 * pick(1, 6);
    thip_value_t y0 = -1, y1 = -1, y2 = -1;
    switch (mode) {
    case 0: return linear(N, result(N, (int)(rng() % 3)), &y0);
    case 1: {
        if (thip_status_t s = linear(N, result(N, (int)(rng() % 3)), &y0)) return s;
        const int64_t N2 = 16 * pick(1, 3);
        if (thip_status_t s = linear(N2, result(N2, (int)(rng() % 3)), &y1)) return s;
        if (rng() & 1) return linear(N2, result(N2, 0), &y2);
        return THIP_OK;
    }
    case 2: {
        const int how = (int)(rng() % 2);
        if (thip_status_t s = linear(N, result(N, how), &y0)) return s;
        if (thip_status_t s = linear(N, result(N, how), &y1)) return s;
        return add(y0, y1, N);
    }
    case 3: {
        if (thip_status_t s = linear(K, result(K, (int)(rng() % 2)), &y0)) return s;  // a residual needs N == K
        return (rng() & 1) ? add(y0, x, K) : add(x, y0, K);
    }
    default: {
        const int64_t B = pick(1, 3), H = pick(1, insane ? 40 : 8), D = 8 * pick(1, 8), T = pick(1, 40);
        const thip_value_t q = binding(p, nextBinding++, {B, H, D}, THIP_DTYPE_BF16);
        const thip_value_t keys = binding(p, nextBinding++, {B, T, D}, THIP_DTYPE_BF16);
        thip_hl_transpose_t t;
        memset(&t, 0, sizeof(t));
        t.rank = 3;
        t.perm[0] = 0; t.perm[1] = 2; t.perm[2] = insane && rng() % 4 == 0 ? wild() : 1;
        t.input = keys;
        int64_t tshape[3] = {B, D, T};
        if (thip_status_t s = thip_program_tensor(p, THIP_DTYPE_BF16, 3, tshape, &t.init)) return s;
        if (thip_status_t s = thip_hl_transpose(p, &t)) return s;
        thip_hl_matmul_t m;
        memset(&m, 0, sizeof(m));
        m.init = binding(p, nextBinding++, {B, H, T}, THIP_DTYPE_BF16);
        m.output_min = noLo;
        m.output_max = noHi;
        m.scale_bias = zero;
        m.input1 = q;
        m.input2 = t.init;
        return thip_hl_matmul(p, &m);
    }
    }
}

// One random program; `insane` also randomises attributes beyond what any pattern would produce.
static bool buildProgram(bool insane, Blob *out, long *statuses) {
    thip_program_t *p = nullptr;
    if (thip_program_create(&p) != THIP_OK) return false;
    if (rng() % 4 == 0) {
        const thip_status_t st = buildDecodeProgram(p, insane);
        statuses[st == THIP_OK ? 0 : 1]++;
        bool have = false;
        if (st == THIP_OK) {
            void *blob = nullptr;
            size_t size = 0;
            const thip_status_t ss = thip_program_serialize(p, &blob, &size);
            statuses[ss == THIP_OK ? 2 : 3]++;
            if (ss == THIP_OK) {
                out->words.assign((size + 7) / 8, 0);
                out->size = size;
                memcpy(out->data(), blob, size);
                thip_blob_free(blob);
                have = true;
            }
        }
        thip_program_destroy(p);
        return have;
    }
    const int64_t N = pick(1, 2), H = pick(1, 9), W = pick(1, 9), C = pick(1, 40), O = pick(1, 40);
    const int64_t KH = pick(1, 3), KW = pick(1, 3);
    const bool nhwc = rng() & 1;
    auto act = [&](int64_t c, int64_t h, int64_t w) { return nhwc ? std::vector<int64_t>{N, h, w, c} : std::vector<int64_t>{N, c, h, w}; };
    uint32_t nextBinding = 0;
    thip_value_t x = binding(p, nextBinding++, act(C, H, W));
    const int kind = (int)(rng() % 7);
    thip_status_t st = THIP_OK;
    auto attr = [&](int32_t sane) { return insane && (rng() % 3 == 0) ? wild() : sane; };
    switch (kind) {
    case 0: {  // conv2d
        const int64_t pl = pick(0, 1), pt = pick(0, 1), OH = H + 2 * pt - KH + 1, OW = W + 2 * pl - KW + 1;
        thip_hl_conv2d_t c;
        memset(&c, 0, sizeof(c));
        c.init = binding(p, nextBinding++, act(O, OH > 0 ? OH : 1, OW > 0 ? OW : 1));
        c.input_zp = attr(-3); c.weight_zp = attr(0); c.output_zp = attr(5); c.output_min = attr(-128); c.output_max = attr(127);
        c.shift_factor = attr((int32_t)pick(0, 45)); c.groups = attr(1);
        c.pad[0] = c.pad[1] = insane ? attr((int32_t)pl) : pl; c.pad[2] = c.pad[3] = pt;
        c.stride[0] = attr(1); c.stride[1] = 1; c.dilation[0] = c.dilation[1] = 1;
        c.nhwc_input = nhwc;
        c.weights = constantI8(p, {O, C, KH, KW});
        c.scale_bias = constantI32(p, (size_t)(insane && rng() % 4 == 0 ? pick(0, 2 * O) : 2 * O));
        c.input = insane && rng() % 5 == 0 ? wild() : x;
        st = thip_hl_conv2d(p, &c);
        break;
    }
    case 1: {  // depthwise
        thip_hl_depthwise_conv2d_t c;
        memset(&c, 0, sizeof(c));
        const int64_t OH = H + 2 - 3 + 1, OW = W + 2 - 3 + 1;
        c.init = binding(p, nextBinding++, act(C, OH, OW));
        c.input_zp = attr(-3); c.output_zp = attr(5); c.output_min = attr(-128); c.output_max = attr(127);
        c.shift_factor = attr((int32_t)pick(0, 45)); c.groups = attr((int32_t)C);
        c.pad[0] = c.pad[1] = c.pad[2] = c.pad[3] = 1;
        c.stride[0] = c.stride[1] = attr(1); c.dilation[0] = c.dilation[1] = 1;
        c.nhwc_input = nhwc;
        c.weights = constantI8(p, {C, 1, 3, 3});
        c.scale_bias = constantI32(p, (size_t)(2 * C));
        c.input = x;
        st = thip_hl_depthwise_conv2d(p, &c);
        break;
    }
    case 2: {  // fully_connected on a separate binding
        const int64_t M = pick(1, 40), K = pick(1, 70), Nn = pick(1, 50);
        thip_hl_fully_connected_t c;
        memset(&c, 0, sizeof(c));
        c.input = binding(p, nextBinding++, {M, K});
        c.init = binding(p, nextBinding++, {M, Nn}, insane && rng() % 4 == 0 ? THIP_DTYPE_I32 : THIP_DTYPE_I8);
        c.input_zp = -128; c.output_zp = attr(1); c.output_min = attr(-128); c.output_max = attr(127);
        c.shift_factor = attr((int32_t)pick(0, 45));
        c.weights = constantI8(p, {Nn, K});
        c.scale_bias = constantI32(p, (size_t)(2 * Nn));
        st = thip_hl_fully_connected(p, &c);
        break;
    }
    case 3: {  // matmul, run-time or constant input2
        const int64_t B = pick(1, 3), M = pick(1, 20), K = pick(1, 40), Nn = pick(1, 30);
        thip_hl_matmul_t c;
        memset(&c, 0, sizeof(c));
        c.input1 = binding(p, nextBinding++, {B, M, K});
        c.input2 = rng() & 1 ? binding(p, nextBinding++, {B, K, Nn}) : constantI8(p, {K, Nn});
        c.init = binding(p, nextBinding++, {B, M, Nn}, THIP_DTYPE_I16);
        c.output_zp = attr(0); c.output_min = attr(-32768); c.output_max = attr(32767); c.shift = attr(0);
        c.scale_bias = constantI32(p, 2);
        st = thip_hl_matmul(p, &c);
        break;
    }
    case 4: {  // maxpool
        thip_hl_maxpool2d_t c;
        memset(&c, 0, sizeof(c));
        const int64_t k = pick(1, 2), OH = (H - k) / k + 1, OW = (W - k) / k + 1;
        c.init = binding(p, nextBinding++, act(C, OH > 0 ? OH : 1, OW > 0 ? OW : 1));
        c.input_zp = attr(-128); c.output_min = attr(-128); c.output_max = attr(127);
        c.stride[0] = c.stride[1] = attr((int32_t)k); c.kernel[0] = c.kernel[1] = attr((int32_t)k);
        c.nhwc_input = nhwc;
        c.weights = THIP_NO_VALUE; c.scale_bias = THIP_NO_VALUE;
        c.input = x;
        st = thip_hl_maxpool2d(p, &c);
        break;
    }
    case 5: {  // global average pool (N,H,W,C)
        thip_hl_avg_pool2d_t c;
        memset(&c, 0, sizeof(c));
        thip_value_t in = binding(p, nextBinding++, {N, H, W, C});
        c.init = binding(p, nextBinding++, {N, 1, 1, C});
        c.input_zp = attr(-3); c.output_zp = attr(2); c.output_min = attr(-128); c.output_max = attr(127); c.shift_factor = attr(20);
        c.weights = THIP_NO_VALUE;
        c.scale_bias = constantI32(p, 2);
        c.input = in;
        st = thip_hl_avg_pool2d(p, &c);
        break;
    }
    default: {  // add
        thip_hl_add_t c;
        memset(&c, 0, sizeof(c));
        c.input1 = x;
        c.input2 = binding(p, nextBinding++, act(C, H, W));
        c.init = binding(p, nextBinding++, act(C, H, W));
        c.name = "add"; c.input_zp = 0; c.output_zp = attr(-2); c.output_min = attr(-128); c.output_max = attr(127); c.shift_factor = attr(12);
        std::vector<int16_t> w2 = {(int16_t)pick(-3000, 3000), (int16_t)pick(-3000, 3000)};
        int64_t two[1] = {2};
        thip_program_constant(p, THIP_DTYPE_I16, 1, two, w2.data(), 4, &c.weights);
        c.scale_bias = constantI32(p, 2);
        st = thip_hl_add(p, &c);
        break;
    }
    }
    statuses[st == THIP_OK ? 0 : 1]++;
    bool have = false;
    if (st == THIP_OK) {
        void *blob = nullptr;
        size_t size = 0;
        const thip_status_t ss = thip_program_serialize(p, &blob, &size);
        statuses[ss == THIP_OK ? 2 : 3]++;
        if (ss == THIP_OK) {
            out->words.assign((size + 7) / 8, 0);
            out->size = size;
            memcpy(out->data(), blob, size);
            thip_blob_free(blob);
            have = true;
        }
    }
    thip_program_destroy(p);
    return have;
}

static void oracleSmoke() {
    for (int it = 0; it < 40; it++) {
        const int N = (int)pick(1, 2), H = (int)pick(1, 7), W = (int)pick(1, 7), C = (int)pick(1, 9), O = (int)pick(1, 9), K = (int)pick(1, 3);
        const int pad = (int)pick(0, 1), OH = H + 2 * pad - K + 1, OW = W + 2 * pad - K + 1;
        if (OH <= 0 || OW <= 0) continue;
        std::vector<int8_t> x((size_t)N * H * W * C), w((size_t)O * C * K * K), y((size_t)N * OH * OW * O);
        std::vector<int32_t> sb(2 * (size_t)O);
        for (auto &v : x) v = (int8_t)rng();
        for (auto &v : w) v = (int8_t)rng();
        for (auto &v : sb) v = (int32_t)pick(1, 1 << 30);
        torq_requant_t rq = {(int32_t)pick(0, 40), 3, -128, 127};
        const int64_t padv[4] = {pad, pad, pad, pad}, stride[2] = {1, 1};
        torq_conv2d(x.data(), w.data(), sb.data(), y.data(), N, C, H, W, O, K, K, padv, stride, -3, &rq, TORQ_LAYOUT_NHWC, 1);
        std::vector<int8_t> fx((size_t)H * C), fw((size_t)O * C), fy((size_t)H * O);
        for (auto &v : fx) v = (int8_t)rng();
        for (auto &v : fw) v = (int8_t)rng();
        torq_fully_connected(fx.data(), fw.data(), sb.data(), fy.data(), H, C, O, &rq, 1);
    }
}

int main(int argc, char **argv) {
    const int programs = argc > 1 ? atoi(argv[1]) : 300, mutations = argc > 2 ? atoi(argv[2]) : 60;
    long statuses[4] = {0, 0, 0, 0}, valid = 0, refused = 0, accepted = 0, grouped = 0;
    for (int it = 0; it < programs; it++) {
        Blob blob;
        const bool insane = it % 3 == 2;
        if (!buildProgram(insane, &blob, statuses)) continue;
        // what the emitter wrote must validate
        if (thip_descriptor_validate(blob.data(), blob.size) != THIP_OK) {
            printf("FAIL: emitter output does not validate: %s\n", thip_status_message());
            return 1;
        }
        valid++;
        const thip::DescHeader *h = (const thip::DescHeader *)blob.data();
        {
            const thip::DescOp *ops = (const thip::DescOp *)(blob.data() + h->ops_offset);
            for (uint32_t i = 0; i < h->op_count; i++) grouped += ops[i].kind == thip::kKindDecLinear || ops[i].kind == thip::kKindDecMatmul;
        }
        const size_t structured = (size_t)h->data_offset;  // header + records + tables: where a flip matters
        for (int m = 0; m < mutations; m++) {
            Blob bad = blob;
            size_t size = bad.size;
            const int how = (int)(rng() % 5);
            if (how == 0) {
                size = (size_t)pick(0, (int64_t)bad.size);  // truncation
            } else {
                const int flips = (int)pick(1, 4);
                for (int f = 0; f < flips; f++) {
                    const size_t at = (size_t)pick(0, (int64_t)(how == 1 ? sizeof(thip::DescHeader) : structured) - 1);
                    if (how == 4) {
                        const int32_t v = wild();  // a whole field replaced
                        memcpy(bad.data() + (at & ~(size_t)3), &v, 4);
                    } else {
                        bad.data()[at] ^= (uint8_t)(1u << (rng() % 8));
                    }
                }
            }
            const thip_status_t s = thip_descriptor_validate(bad.data(), size);
            (s == THIP_OK ? accepted : refused)++;
            char fmt[32];
            size_t inferred = 0;
            (void)thip_infer_format(bad.data(), size, sizeof(fmt), fmt, &inferred);
        }
    }
    oracleSmoke();
    printf("programs built %ld (refused by the emitter %ld), serialised %ld (refused %ld), valid blobs %ld (grouped-linear / in-place-matmul records %ld), mutants refused %ld / accepted %ld\n",
           statuses[0], statuses[1], statuses[2], statuses[3], valid, grouped, refused, accepted);
    if (valid < programs / 4 || refused == 0 || (programs >= 200 && grouped == 0)) {
        printf("FAIL: the fuzz did not reach both outcomes\n");
        return 1;
    }
    printf("fuzz ok\n");
    return 0;
}
