"""ctypes bindings of the CPU oracle (oracle/liboracle.so) and, where it was built, of the reference's own C
oracles (oracle/_ref/libref.so). Test support only: nothing under anemone_amd/ imports this."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

u8p = C.POINTER(C.c_uint8)
u16p = C.POINTER(C.c_uint16)
u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)


def ptr(array, kind):
    assert array.flags["C_CONTIGUOUS"]
    return array.ctypes.data_as(kind)


def _load_oracle():
    path = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-s"])
    lib = C.CDLL(path)
    u32, f32, i32, vp = C.c_uint32, C.c_float, C.c_int, C.c_void_p
    sig = {
        "orc_exl3_bits_x2": (u32, [u32]),
        "orc_exl3_window_end": (u32, [u32, u32]),
        "orc_exl3_matrix_bytes": (C.c_uint64, [u32, u32, u32]),
        "orc_exl3_code_bytes": (C.c_uint64, [u32, u32, u32]),
        "orc_exl3_codebook": (C.c_uint16, [u32]),
        "orc_exl3_position": (u32, [u32, u32]),
        "orc_exl3_place": (None, [u32, u32p, u32p]),
        "orc_exl3_tile_states": (None, [u32, u32p, u16p]),
        "orc_exl3_states": (None, [u8p, u32, u32, u32, u16p]),
        "orc_exl3_decode_matrix": (None, [u8p, u32, u32, u32, u16p]),
        "orc_h128_f32": (None, [f32p]),
        "orc_h128_f64": (None, [f64p, f64p]),
        "orc_expf": (f32, [f32]),
        "orc_exl3_operand": (None, [u16p, u16p, u32, u16p]),
        "orc_exl3_product": (None, [u16p, u32, u32, u16p, u32, i32, f32p]),
        "orc_exl3_product_codes": (None, [u8p, u32, u32, u32, u16p, u32, f32p]),
        "orc_exl3_activate": (None, [f32p, f32p, u16p, u16p, u16p, u32, f32, u16p, u16p]),
        "orc_exl3_finish": (None, [f32p, u16p, u32, f32, f32p]),
        "orc_exl3_row_sum": (None, [f32p, u32, u32, u32, f32p]),
        "orc_exl3_linear_f64": (None, [u8p, u32, u32, u32, f64p, f64p]),
        "orc_exl3_moe_layer": (None, [u16p, u32, u32, u32, u32, u32p, f32p, u32, C.POINTER(vp), u8p, f32, f32p,
                                      u16p, f32p, u32]),
        "orc_log1pf": (f32, [f32]),
        "orc_router_affinity": (f32, [f32, i32]),
        "orc_router_projection": (None, [u16p, u16p, u32, u32, u32, f32p]),
        "orc_router_select": (None, [f32p, f32p, u32, u32, i32, f32, u32p, f32p]),
        "orc_router_route": (None, [u16p, u16p, f32p, u32, u32, u32, u32, i32, i32, f32, f32p, u32p, f32p]),
        "orc_router_jobs": (None, [u32p, f32p, u32, u32, u32, u32, u64p, vp]),
        "orc_router_wide_tile_count": (u32, [u32, u32, u32]),
        "orc_router_wide_job_count": (u32, [u32, u32, u32]),
        "orc_router_wide_sort": (None, [u32p, f32p, u32, u32, u32, u32, u64p, vp, vp, vp]),
        "orc_router_wide_jobs": (None, [u32p, f32p, u32, u32, u32, u32, u64p, vp]),
        "orc_linear_stored_bytes": (C.c_uint64, [i32, u32, u32]),
        "orc_linear_scale_count": (C.c_uint64, [i32, u32, u32]),
        "orc_linear_lay_out": (i32, [i32, u32, u32, u8p, u8p, u8p]),
        "orc_linear_read": (i32, [i32, u32, u32, u8p, u32, u32, u32p, u32p]),
        "orc_act_quantize": (i32, [u16p, u32, u8p, u8p]),
        "orc_codes_lane_order": (None, [u8p, u32, u8p]),
        "orc_operands_lay_out": (None, [u8p, u8p, u32, u16p]),
        "orc_linear_products": (i32, [i32, u32, u32, u8p, u32, u32, u8p, u8p, u32, f64p, f64p]),
        "orc_linear_products_128": (i32, [u32, u32, u8p, u32, u32, u8p, f32p, u32, f64p, f64p]),
        "orc_linear_products_128_of": (i32, [i32, u32, u32, u8p, u32, u32, u8p, f32p, u32, f64p, f64p]),
        "orc_linear_within_tolerance": (i32, [C.c_uint16, C.c_double, C.c_double, u32, u32]),
        "orc_linear_within_allowance": (i32, [C.c_uint16, C.c_double, C.c_double, u32, u32, C.c_double]),
        "orc_hidden_value": (C.c_double, [C.c_double] * 4),
        "orc_hidden_bits": (C.c_uint16, [f32] * 4),
        "orc_row_sum_bf16": (f32, [u16p, u32, u32, u32]),
        "orc_act_quantize_128": (None, [u16p, u32, u8p, f32p]),
        "orc_fp8_block128_products": (None, [u32, u32, u8p, f32p, u8p, f32p, u32, f64p]),
        "orc_linear_moe_layer": (None, [i32, u16p, u32, u32, u32, u32, u32p, f32p, u32, C.POINTER(vp), f32, f32p,
                                        u16p, u16p, u32]),
        "orc_hyper_post": (None, [u16p, f32p, f32p, u16p, f32p, u32, u16p]),
        "orc_expert_join": (None, [u16p, u16p, u16p, f32p, f32p, f32p, u32, u32, u32]),
        "orc_trunk_hidden": (None, [u16p, u16p, f32, u32, u16p]),
        "orc_reciprocal_root": (f32, [f32]),
        "orc_dense_linear": (i32, [u32, vp, u32, u32, u32, f32, f32, u32, u16p, u32, vp]),
        "orc_hyper_sinkhorn": (None, [f32p, f32p, f32p, f32p, f32p, f32p]),
        "orc_hyper_mix_finish": (None, [u16p, f32p, f32p, f32p, f32p, u16p, u32, f32p, f32p, u16p]),
        "orc_hyper_collapse": (None, [u16p, f32p, u32, u16p]),
        "orc_hyper_norm_operand": (f32, [u16p, u32]),
        "orc_hyper_norm_with": (None, [u16p, u16p, f32, u32, u16p]),
    }
    for name, (restype, argtypes) in sig.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def _load_ref():
    path = os.path.join(ORACLE_DIR, "_ref", "libref.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path)
    u32, f32 = C.c_uint32, C.c_float
    lib.test_exl3_codebook.restype = C.c_uint16
    lib.test_exl3_codebook.argtypes = [u32]
    lib.test_exl3_position.restype = u32
    lib.test_exl3_position.argtypes = [u32, u32]
    lib.test_exl3_state.restype = C.c_uint16
    lib.test_exl3_state.argtypes = [u8p, u32, u32, u32, u32, u32]
    lib.test_exl3_decode_matrix.restype = None
    lib.test_exl3_decode_matrix.argtypes = [u8p, u32, u32, u32, u16p]
    lib.test_exl3_chain.restype = None
    lib.test_exl3_chain.argtypes = [u32, u16p, u32, u32, u32, u16p, u32, f32p]
    lib.test_router_affinity.restype = C.c_double
    lib.test_router_affinity.argtypes = [f32]
    lib.test_router_affinity_holds.restype = C.c_bool
    lib.test_router_affinity_holds.argtypes = [f32, f32]
    lib.test_router_select.restype = None
    lib.test_router_select.argtypes = [f32p, f32p, C.c_bool, u32p, f32p]
    lib.test_router_jobs.restype = None
    lib.test_router_jobs.argtypes = [u32p, f32p, u32, u32, u64p, C.c_void_p]
    lib.test_router_wide_sort.restype = None
    lib.test_router_wide_sort.argtypes = [u32p, f32p, u32, u32, u64p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.test_router_wide_jobs.restype = None
    lib.test_router_wide_jobs.argtypes = [u32p, f32p, u32, u32, u64p, C.c_void_p]
    lib.test_weight_format_lay_out.restype = C.c_int
    lib.test_weight_format_lay_out.argtypes = [C.c_int, C.c_void_p, u8p, C.c_uint64, u8p, C.c_uint64, u8p, C.c_uint64]
    lib.test_weight_format_read_weight.restype = C.c_int
    lib.test_weight_format_read_weight.argtypes = [C.c_int, C.c_void_p, u8p, C.c_uint64, u32, u32, C.c_void_p]
    lib.test_linear_quantize.restype = C.c_int
    lib.test_linear_quantize.argtypes = [u16p, u32, u8p, u8p]
    lib.test_linear_codes_lay_out.restype = C.c_int
    lib.test_linear_codes_lay_out.argtypes = [u8p, u32, u8p]
    lib.test_linear_operands_lay_out.restype = C.c_int
    lib.test_linear_operands_lay_out.argtypes = [u8p, u8p, u32, u16p]
    lib.test_linear_products.restype = C.c_int
    lib.test_linear_products.argtypes = [C.c_int, C.c_void_p, u8p, C.c_uint64, u32, u32, f64p, u8p, u32, u32,
                                         C.c_void_p]
    lib.test_linear_fed_values_of_codes.restype = C.c_int
    lib.test_linear_fed_values_of_codes.argtypes = [u8p, u32, f64p]
    lib.test_linear_hidden_value.restype = C.c_double
    lib.test_linear_hidden_value.argtypes = [C.c_double] * 4
    lib.test_linear_row_sum.restype = f32
    lib.test_linear_row_sum.argtypes = [u16p, u32, u32, u32]
    lib.test_linear_output_is_within_tolerance.restype = C.c_bool
    lib.test_linear_output_is_within_tolerance.argtypes = [C.c_uint16, C.c_void_p, u32, u32]
    if hasattr(lib, "test_hyper_post"):
        lib.test_hyper_post.restype = None
        lib.test_hyper_post.argtypes = [u16p, f32p, f32p, u16p, f32p, u16p]
        lib.test_hyper_sinkhorn.restype = None
        lib.test_hyper_sinkhorn.argtypes = [f32p, f32p, f32p, f32p, f32p, f32p]
        lib.test_hyper_collapse.restype = None
        lib.test_hyper_collapse.argtypes = [u16p, f32p, u16p]
        lib.test_hyper_norm_operand.restype = f32
        lib.test_hyper_norm_operand.argtypes = [u16p]
        lib.test_hyper_reciprocal_root.restype = f32
        lib.test_hyper_reciprocal_root.argtypes = [f32]
        lib.test_hyper_norm_with.restype = None
        lib.test_hyper_norm_with.argtypes = [u16p, u16p, f32, u16p]
        lib.test_hyper_float_places.restype = u32
        lib.test_hyper_float_places.argtypes = [f32, f32]
    if hasattr(lib, "test_dense_reference"):
        lib.test_dense_reference.restype = None
        lib.test_dense_reference.argtypes = [u32, C.c_void_p, u32, u32, f32, u16p, u32, u32, u32, f64p, f64p]
        lib.test_dense_output_holds.restype = C.c_bool
        lib.test_dense_output_holds.argtypes = [u32, f32, C.c_void_p, C.c_uint64, C.c_double, C.c_double]
    return lib


orc = _load_oracle()
ref = _load_ref()


class Shape(C.Structure):  # struct matrix_shape_record of the reference
    _fields_ = [("output_size", C.c_uint32), ("input_size", C.c_uint32), ("bits_per_weight", C.c_uint32),
                ("reserved", C.c_uint32)]


JOB_DTYPE = np.dtype([("gate_offset", "<u8"), ("up_offset", "<u8"), ("down_offset", "<u8"), ("row_count", "<u4"),
                      ("expert", "<u4"), ("pair_index", "<u4", (8,)), ("route_weight", "<f4", (8,))])
PAIR_DTYPE = np.dtype([("pair_index", "<u4"), ("route_weight", "<f4")])
RUN_DTYPE = np.dtype([("first_pair", "<u4"), ("pair_count", "<u4")])
TILE_DTYPE = np.dtype([("gate_offset", "<u8"), ("up_offset", "<u8"), ("down_offset", "<u8"), ("first_pair", "<u4"),
                       ("pair_count", "<u4")])
assert JOB_DTYPE.itemsize == 96 and TILE_DTYPE.itemsize == 32


# ---- the seeded generator of every synthetic tensor ----

def splitmix_words(seed, count):
    """`count` 64-bit outputs of splitmix64 from `seed`, vectorised."""
    with np.errstate(over="ignore"):
        steps = (np.arange(1, count + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)) + np.uint64(seed)
        z = steps
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform01(seed, count):
    return (splitmix_words(seed, count) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def normals(seed, count):
    """Box-Muller on two draws each, computed in double."""
    n = (count + 1) // 2
    u = uniform01(seed, 2 * n)
    u1, u2 = np.maximum(u[:n], 1e-300), u[n:]
    r = np.sqrt(-2.0 * np.log(u1))
    return np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:count]


def to_bf16(values):
    bits = np.asarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def exl3_matrix(seed, inputs, outputs, stored_width):
    """One stored EXL3 matrix: uniform random codes, suh = +-1, svh = +-U(0.5,1.5)/64 (fp16)."""
    code_bytes = int(orc.orc_exl3_code_bytes(inputs, outputs, stored_width))
    codes = splitmix_words(seed, code_bytes // 8).view(np.uint8)
    signs = splitmix_words(seed ^ 0xABCDEF, inputs + outputs)
    suh = np.where(signs[:inputs] & np.uint64(1), 1.0, -1.0).astype(np.float16)
    magnitude = (0.5 + uniform01(seed ^ 0x123457, outputs)) / 64.0
    svh = (np.where(signs[inputs:] & np.uint64(1), 1.0, -1.0) * magnitude).astype(np.float16)
    return np.concatenate([codes, suh.view(np.uint8), svh.view(np.uint8)])
