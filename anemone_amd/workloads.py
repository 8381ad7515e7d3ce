"""Seeded synthetic tensors of the benchmark configurations: one generator (splitmix64) for everything, normals by
Box-Muller in double precision, rounded once. Numpy only; used by bench.py, the smoke run and the tests."""
import numpy as np

SEED = 0x5EED0000


def splitmix_words(seed, count):
    with np.errstate(over="ignore"):
        z = (np.arange(1, count + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)) + np.uint64(seed)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform01(seed, count):
    return (splitmix_words(seed, count) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def normals(seed, count):
    n = (count + 1) // 2
    u = uniform01(seed, 2 * n)
    r = np.sqrt(-2.0 * np.log(np.maximum(u[:n], 1e-300)))
    return np.concatenate([r * np.cos(2 * np.pi * u[n:]), r * np.sin(2 * np.pi * u[n:])])[:count]


def to_bf16(values):
    bits = np.asarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def exl3_bits_x2(stored_width):
    return 2 * stored_width if 1 <= stored_width <= 8 else stored_width // 8


def exl3_matrix_bytes(inputs, outputs, stored_width):
    return inputs * outputs // 16 * exl3_bits_x2(stored_width) + 2 * (inputs + outputs)


def exl3_matrix(seed, inputs, outputs, stored_width):
    """One stored EXL3 matrix: uniform random codes (every bit pattern is a tile), suh = +-1,
    svh = +-U(0.5, 1.5) / 64 rounded to fp16."""
    code_bytes = inputs * outputs // 16 * exl3_bits_x2(stored_width)
    codes = splitmix_words(seed, code_bytes // 8).view(np.uint8)
    signs = splitmix_words(seed ^ 0xABCDEF, inputs + outputs)
    suh = np.where(signs[:inputs] & np.uint64(1), 1.0, -1.0).astype(np.float16)
    magnitude = (0.5 + uniform01(seed ^ 0x123457, outputs)) / 64.0
    svh = (np.where(signs[inputs:] & np.uint64(1), 1.0, -1.0) * magnitude).astype(np.float16)
    return np.concatenate([codes, suh.view(np.uint8), svh.view(np.uint8)])


def exl3_moe_layer(config, hidden, inner, expert_count, width_choices=(2, 3, 4), probabilities=(0.30, 0.50, 0.20)):
    """Widths [E][3] drawn per tensor and the experts' stored matrices; router weights bf16 N(0, 0.02)."""
    base = SEED + (config << 20)
    draws = uniform01(base + 1, expert_count * 3)
    edges = np.cumsum(probabilities)
    widths = np.array(width_choices, dtype=np.uint32)[np.minimum(np.searchsorted(edges, draws, side="right"), len(width_choices) - 1)]
    widths = widths.reshape(expert_count, 3)
    matrices = []
    for e in range(expert_count):
        matrices.append([exl3_matrix(base + 16 + 3 * e + 0, hidden, inner, int(widths[e, 0])),
                         exl3_matrix(base + 16 + 3 * e + 1, hidden, inner, int(widths[e, 1])),
                         exl3_matrix(base + 16 + 3 * e + 2, inner, hidden, int(widths[e, 2]))])
    router = to_bf16(normals(base + 2, expert_count * hidden) * 0.02).reshape(expert_count, hidden)
    return widths, matrices, router


def activations(config, rows, hidden):
    return to_bf16(normals(SEED + (config << 20) + 3, rows * hidden)).reshape(rows, hidden)


def e2m1_lay_out(codes, scales):
    """codes uint8 [outputs][inputs] (0..15), scales uint8 [outputs][inputs / 32] -> the stored bytes of
    WEIGHT_FORMAT_E2M1_SCALED: words [tile][load][lane][step] (nibble at bit 4 r + 16 h of a word is
    W[16 tile + g + 8 (r % 2)][64 load + 16 step + 2 t + 8 (r / 2) + h], lane = 4 g + t), then the scales
    [tile][load][g] (byte 2 q + r: inputs 64 load + 32 q.. of output 16 tile + g + 8 r)."""
    outputs, inputs = codes.shape
    tiles, loads = outputs // 16, inputs // 64
    # w[tile, r%2, g, load, step, r/2, t, h]
    w = codes.reshape(tiles, 2, 8, loads, 4, 2, 4, 2).astype(np.uint32)
    words = np.zeros((tiles, loads, 8, 4, 4), dtype=np.uint32)  # [tile][load][g][t][step]
    for r in range(4):
        for h in range(2):
            words |= w[:, r % 2, :, :, :, r // 2, :, h].transpose(0, 2, 1, 4, 3) << np.uint32(4 * r + 16 * h)
    s = scales.reshape(tiles, 2, 8, loads, 2)  # [tile][r][g][load][q]
    scale_bytes = s.transpose(0, 3, 2, 4, 1)    # [tile][load][g][q][r]
    return np.concatenate([words.reshape(-1).view(np.uint8), np.ascontiguousarray(scale_bytes).reshape(-1)])


def fp4_matrix(seed, outputs, inputs, scale_code=120):
    """Uniform random E2M1 codes with E8M0 scales scale_code + {0, 1}: weights of standard deviation about 0.02."""
    raw = splitmix_words(seed, outputs * inputs // 16)
    codes = ((raw[:, None] >> (np.arange(16, dtype=np.uint64) * np.uint64(4))) & np.uint64(15)).astype(np.uint8).reshape(outputs, inputs)
    scales = (scale_code + (splitmix_words(seed ^ 0x5CA1E, outputs * inputs // 32) & np.uint64(1))).astype(np.uint8).reshape(outputs, inputs // 32)
    return e2m1_lay_out(codes, scales)


def e4m3_lay_out(codes, scales):
    """codes uint8 [outputs][inputs] (E4M3 bytes), scales uint8 [ceil(outputs / 32)][inputs / 32] -> the stored bytes of
    WEIGHT_FORMAT_E4M3_SCALED: bytes [tile][group][lane = 4 G + t][16], byte b of a lane is
    W[16 tile + G + 8 (b % 2)][32 group + 8 (b / 4) + 2 t + (b / 2) % 2]; then the scales as they are."""
    outputs, inputs = codes.shape
    tiles, groups = outputs // 16, inputs // 32
    # w[tile, b%2, G, group, b/4, t, (b/2)%2]
    w = codes.reshape(tiles, 2, 8, groups, 4, 4, 2)
    stored = w.transpose(0, 3, 2, 5, 4, 6, 1)  # [tile][group][G][t][b/4][(b/2)%2][b%2]
    return np.concatenate([np.ascontiguousarray(stored).reshape(-1), np.ascontiguousarray(scales).reshape(-1)])


def fp8_matrix_of_random_codes(seed, outputs, inputs, scale_code=113):
    """Uniformly random E4M3 codes (every exponent as likely as any other; no NaN code) with E8M0 scales scale_code +
    {0, 1} per 32 x 32 block: a stress of a sum's dynamic range, not a likeness of weights."""
    raw = splitmix_words(seed, outputs * inputs // 8).view(np.uint8).reshape(outputs, inputs)
    codes = np.where((raw & 0x7F) == 0x7F, raw & 0x80, raw).astype(np.uint8)
    rows = (outputs + 31) // 32
    scales = (scale_code + (splitmix_words(seed ^ 0x5CA1E, rows * inputs // 32) & np.uint64(1))).astype(np.uint8).reshape(rows, inputs // 32)
    return e4m3_lay_out(codes, scales)


E4M3_MAGNITUDES = np.array([(m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
                            for e in range(16) for m in range(8)][:127])


def e4m3_nearest(values):
    """Round-to-nearest-even E4M3 codes of float64 values, magnitudes clamped to 448."""
    magnitudes = np.minimum(np.abs(values), 448.0)
    middles = (E4M3_MAGNITUDES[:-1] + E4M3_MAGNITUDES[1:]) / 2.0
    below = np.searchsorted(middles, magnitudes, side="left")   # a tie falls to the lower code here
    tie = (below < 126) & (magnitudes == middles[np.minimum(below, 125)])
    codes = np.where(tie & (below % 2 == 1), below + 1, below).astype(np.uint8)  # of two equally near, the even code
    return codes | (np.signbit(values).astype(np.uint8) << 7)


def fp8_matrix(seed, outputs, inputs, deviation=0.02):
    """Weights N(0, deviation) as WEIGHT_FORMAT_E4M3_SCALED stores them: for every 32 x 32 block the smallest power of two
    that brings the block's largest magnitude to at most 448, and the nearest E4M3 code of each weight over it."""
    assert outputs % 32 == 0 and inputs % 32 == 0
    weights = normals(seed, outputs * inputs).reshape(outputs // 32, 32, inputs // 32, 32) * deviation
    largest = np.maximum(np.abs(weights).max(axis=(1, 3)), 1e-30)
    exponents = np.ceil(np.log2(largest / 448.0)).astype(np.int64)
    codes = e4m3_nearest(weights / (2.0 ** exponents)[:, None, :, None]).reshape(outputs, inputs)
    return e4m3_lay_out(codes, (exponents + 127).astype(np.uint8))


def fp8_block128_matrix(seed, outputs, inputs, deviation=0.02):
    """Weights N(0, deviation) as WEIGHT_FORMAT_E4M3_BLOCK128 stores them: for every 128 x 128 block one float32 scale,
    the block's largest magnitude over 448, and the nearest E4M3 code of each weight over it (a float32 division); the
    codes in WEIGHT_FORMAT_E4M3_SCALED's lane order, the scales float32 [outputs / 128][inputs / 128] behind them."""
    assert outputs % 128 == 0 and inputs % 128 == 0
    weights = (normals(seed, outputs * inputs).reshape(outputs // 128, 128, inputs // 128, 128) * deviation).astype(np.float32)
    scales = (np.maximum(np.abs(weights).max(axis=(1, 3)), np.float32(1e-30)) / np.float32(448.0)).astype(np.float32)
    scaled = (weights / scales[:, None, :, None]).astype(np.float32)
    codes = e4m3_nearest(scaled.astype(np.float64)).reshape(outputs, inputs)
    return e4m3_lay_out(codes, scales.view(np.uint8))


def fp4_moe_layer(config, hidden, inner, expert_count):
    base = SEED + (config << 20)
    matrices = [[fp4_matrix(base + 16 + 3 * e + 0, inner, hidden), fp4_matrix(base + 16 + 3 * e + 1, inner, hidden),
                 fp4_matrix(base + 16 + 3 * e + 2, hidden, inner)] for e in range(expert_count)]
    router = to_bf16(normals(base + 2, expert_count * hidden) * 0.02).reshape(expert_count, hidden)
    return matrices, router
