"""ctypes/numpy front end of the CPU oracle (``liboracle.so``).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by ``bench.py``'s cpu_baseline leg.  Nothing under ``sphconv_amd/`` imports it.

Every function takes and returns numpy arrays in the reference's layouts
(feature [N,C] float32, z_idx [N] int32, z_ptr [B,S0,S1] int32 inclusive scan,
rules [NTile,KV,2,tile_n_max] int32 padded with -1, rule_size [NTile,KV]).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class Geom(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("B", "S0", "S1", "S2", "O0", "O1", "O2", "K0", "K1", "K2",
                 "s0", "s1", "s2", "p0", "p1", "p2", "d0", "d1", "d2", "T0", "T1")]


def build(force: bool = False) -> str:
    so = os.path.join(_HERE, "liboracle.so")
    src = os.path.join(_HERE, "sphconv_oracle.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        _LIB = C.CDLL(so)
        _LIB.orc_tile_n_max.restype = C.c_int
        _LIB.orc_in_tile_size.restype = C.c_int
        _LIB.orc_out_spatial_dim.restype = C.c_int
        _LIB.orc_num_threads.restype = C.c_int
    return _LIB


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def num_threads() -> int:
    return lib().orc_num_threads()


def set_num_threads(n: int):
    lib().orc_set_num_threads(int(n))


def out_spatial(in_shape, kernel, stride, padding, dilation=(1, 1, 1)):
    L = lib()
    return [L.orc_out_spatial_dim(int(i), int(k), int(s), int(p), int(d))
            for i, k, s, p, d in zip(in_shape, kernel, stride, padding, dilation)]


def tile_n_max(B, in_shape, kernel, stride, tile, nnz) -> int:
    L = lib()
    it0 = L.orc_in_tile_size(int(tile[0]), int(stride[0]), int(kernel[0]))
    it1 = L.orc_in_tile_size(int(tile[1]), int(stride[1]), int(kernel[1]))
    return L.orc_tile_n_max(it0, it1, int(B), int(in_shape[0]), int(in_shape[1]),
                            int(in_shape[2]), int(nnz))


def make_geom(B, in_shape, out_shape, kernel, stride, padding, dilation=(1, 1, 1), tile=(2, 2)):
    return Geom(int(B), *map(int, in_shape), *map(int, out_shape), *map(int, kernel),
                *map(int, stride), *map(int, padding), *map(int, dilation), *map(int, tile))


def init_tensor(feature, indices, B, shape):
    """-> (out_feature, z_idx, z_ptr, permutation); fibers sorted by S2."""
    feature = _f32(feature)
    indices = _i32(indices)
    n, c = feature.shape
    S0, S1, S2 = map(int, shape)
    out = np.empty_like(feature)
    z_idx = np.empty(n, np.int32)
    z_ptr = np.empty((B, S0, S1), np.int32)
    perm = np.empty(n, np.int32)
    rc = lib().orc_init_tensor(_p(feature), _p(indices), n, c, int(B), S0, S1, S2,
                               _p(out), _p(z_idx), _p(z_ptr), _p(perm))
    if rc:
        raise ValueError({-1: "coordinate out of range", -2: "duplicate coordinate",
                          -3: "out of memory"}[rc])
    return out, z_idx, z_ptr, perm


def init_tensor_backward(d_out, perm):
    d_out = _f32(d_out)
    perm = _i32(perm)
    res = np.empty_like(d_out)
    lib().orc_init_tensor_backward(_p(d_out), _p(perm), d_out.shape[0], d_out.shape[1], _p(res))
    return res


def to_dense(feature, z_idx, z_ptr, S2):
    """-> [B,S0,S1,S2,C] float32, zeros where inactive."""
    feature, z_idx, z_ptr = _f32(feature), _i32(z_idx), _i32(z_ptr)
    B, S0, S1 = z_ptr.shape
    out = np.zeros((B, S0, S1, int(S2), feature.shape[1]), np.float32)
    lib().orc_to_dense(_p(feature), _p(z_idx), _p(z_ptr), B, S0, S1, int(S2),
                       feature.shape[1], _p(out))
    return out


def to_dense_backward(d_out, z_idx, z_ptr):
    d_out, z_idx, z_ptr = _f32(d_out), _i32(z_idx), _i32(z_ptr)
    B, S0, S1, S2, c = d_out.shape
    res = np.zeros((z_idx.shape[0], c), np.float32)
    lib().orc_to_dense_backward(_p(d_out), _p(z_idx), _p(z_ptr), B, S0, S1, S2, c, _p(res))
    return res


def get_rules_subm(z_idx, z_ptr, B, in_shape, out_shape, kernel, stride, padding,
                   dilation=(1, 1, 1), tile=(2, 2), n_max=None, canonical=True):
    """-> (z_idx, z_ptr, rules, rule_size, dropped)."""
    z_idx, z_ptr = _i32(z_idx), _i32(z_ptr)
    g = make_geom(B, in_shape, out_shape, kernel, stride, padding, dilation, tile)
    kv = int(np.prod(kernel))
    ntile = -(-out_shape[0] // tile[0]) * -(-out_shape[1] // tile[1])
    if n_max is None:
        n_max = tile_n_max(B, in_shape, kernel, stride, tile, z_idx.shape[0])
    grid = np.empty(int(B) * int(np.prod(out_shape)), np.int32)
    rules = np.empty((ntile, kv, 2, n_max), np.int32)
    rule_size = np.empty((ntile, kv), np.int32)
    lib().orc_rules_subm.restype = C.c_int
    dropped = lib().orc_rules_subm(_p(z_idx), _p(z_ptr), C.byref(g), int(n_max),
                                   _p(grid), _p(rules), _p(rule_size))
    if canonical:
        lib().orc_rules_canonicalize(_p(rules), _p(rule_size), ntile, kv, int(n_max))
    return z_idx, z_ptr, rules, rule_size, dropped


def get_rules(z_idx, z_ptr, B, in_shape, out_shape, kernel, stride, padding,
              dilation=(1, 1, 1), tile=(2, 2), n_max=None, canonical=True):
    """-> (oz_idx, oz_ptr, rules, rule_size, dropped)."""
    z_idx, z_ptr = _i32(z_idx), _i32(z_ptr)
    g = make_geom(B, in_shape, out_shape, kernel, stride, padding, dilation, tile)
    kv = int(np.prod(kernel))
    ntile = -(-out_shape[0] // tile[0]) * -(-out_shape[1] // tile[1])
    if n_max is None:
        n_max = tile_n_max(B, in_shape, kernel, stride, tile, z_idx.shape[0])
    grid = np.empty(int(B) * int(np.prod(out_shape)), np.int32)
    oz_ptr = np.empty((int(B), int(out_shape[0]), int(out_shape[1])), np.int32)
    L = lib()
    L.orc_rules_std_outgrid.restype = C.c_int
    L.orc_rules_std_fill.restype = C.c_int
    out_nnz = L.orc_rules_std_outgrid(_p(z_idx), _p(z_ptr), C.byref(g), _p(grid), _p(oz_ptr))
    oz_idx = np.empty(out_nnz, np.int32)
    rules = np.empty((ntile, kv, 2, n_max), np.int32)
    rule_size = np.empty((ntile, kv), np.int32)
    dropped = L.orc_rules_std_fill(_p(z_idx), _p(z_ptr), C.byref(g), int(n_max), _p(grid),
                                   _p(oz_idx), _p(rules), _p(rule_size))
    if canonical:
        L.orc_rules_canonicalize(_p(rules), _p(rule_size), ntile, kv, int(n_max))
    return oz_idx, oz_ptr, rules, rule_size, dropped


def rule_conv(feature, weight, rules, rule_size, out_nnz):
    """fp32 forward; weight [KV,iC,oC]."""
    feature, weight = _f32(feature), _f32(weight)
    rules, rule_size = _i32(rules), _i32(rule_size)
    ntile, kv, _, n_max = rules.shape
    ic, oc = weight.shape[1], weight.shape[2]
    out = np.empty((int(out_nnz), oc), np.float32)
    lib().orc_rule_conv_f32(_p(feature), _p(weight), _p(rules), _p(rule_size), ntile, kv,
                            n_max, ic, oc, int(out_nnz), _p(out))
    return out


def rule_conv_d_feature(d_out, weight_oc_ic, rules, rule_size, tile_grid_shape, nnz):
    """fp32 dgrad; weight already permuted to [KV,oC,iC] as the reference's caller does."""
    d_out, w = _f32(d_out), _f32(weight_oc_ic)
    rules, rule_size = _i32(rules), _i32(rule_size)
    _, kv, _, n_max = rules.shape
    oc, ic = w.shape[1], w.shape[2]
    res = np.empty((int(nnz), ic), np.float32)
    lib().orc_rule_conv_dfeature_f32(_p(d_out), _p(w), _p(rules), _p(rule_size),
                                     int(tile_grid_shape[0]), int(tile_grid_shape[1]), kv,
                                     n_max, ic, oc, int(nnz), _p(res))
    return res


def rule_conv_d_weight(feature, d_out, rules, rule_size):
    feature, d_out = _f32(feature), _f32(d_out)
    rules, rule_size = _i32(rules), _i32(rule_size)
    ntile, kv, _, n_max = rules.shape
    ic, oc = feature.shape[1], d_out.shape[1]
    res = np.empty((kv, ic, oc), np.float32)
    lib().orc_rule_conv_dweight_f32(_p(feature), _p(d_out), _p(rules), _p(rule_size), ntile,
                                    kv, n_max, ic, oc, _p(res))
    return res


def rule_conv_backward(d_out, feature, weight_oc_ic, rules, rule_size, tile_grid_shape):
    """rule_conv.cu:577-597 -> (d_feature, d_weight[KV,iC,oC])."""
    d_feature = rule_conv_d_feature(d_out, weight_oc_ic, rules, rule_size, tile_grid_shape,
                                    feature.shape[0])
    d_weight = rule_conv_d_weight(feature, d_out, rules, rule_size)
    return d_feature, d_weight


def rule_conv_i8(feature, weight, scale, rules, rule_size, out_nnz, return_acc=False):
    feature = np.ascontiguousarray(feature, dtype=np.int8)
    weight = np.ascontiguousarray(weight, dtype=np.int8)
    scale = _f32(scale)
    rules, rule_size = _i32(rules), _i32(rule_size)
    ntile, kv, _, n_max = rules.shape
    ic, oc = weight.shape[1], weight.shape[2]
    out = np.empty((int(out_nnz), oc), np.int8)
    acc = np.empty((int(out_nnz), oc), np.int32)
    lib().orc_rule_conv_i8(_p(feature), _p(weight), _p(scale), _p(rules), _p(rule_size), ntile,
                           kv, n_max, ic, oc, int(out_nnz), _p(acc), _p(out))
    return (out, acc) if return_acc else out


def xyz2rangevoxel(points, v_res=64, h_res=512, d_res=512, v_range=(87.5, 103.4), h_range=(-45, 45),
                   d_range=(6, 70.4), log=True):
    """numpy restatement of xyz2RangeVoxel (reference sphconv/data.py:75-128) for float32 points.
    The reference mixes float32 arrays with float64 numpy scalars; under the promotion rules of
    the numpy it was written for, each scalar enters the float32 operation rounded to float32 --
    written out here with explicit float32 casts so that the result does not depend on the numpy
    version.  Returns (feature [1,C,1,V,H], depth [1,1,V,H] int32, thick [1,V,H] int32,
    per-point (theta, phi, depth) bins [M,3] int32 and the unclamped float bins [M,3])."""
    f32 = np.float32
    pts = np.ascontiguousarray(points, dtype=np.float32)
    x, y, z = pts[:, 0], pts[:, 1], pts[:, 2]
    channel = pts.shape[1]
    with np.errstate(all="ignore"):
        x2y2 = x * x + y * y                                   # data.py:80
        r = np.sqrt(x2y2 + z * z)                              # :81
        thetas = np.arccos(z / r)                              # :82
        phis = np.arcsin(y / np.sqrt(x2y2))                    # :83
        delta_phi = f32(np.radians(h_range[1] - h_range[0]) / h_res)      # :85
        delta_theta = f32(np.radians(v_range[1] - v_range[0]) / v_res)    # :86
        tf = (thetas - f32(np.radians(v_range[0]))) / delta_theta         # :88
        pf = (phis - f32(np.radians(h_range[0]))) / delta_phi             # :89
        if log:
            delta_r = f32((np.log(d_range[1]) - np.log(d_range[0])) / d_res)   # :92
            df = (np.log(r) - f32(np.log(d_range[0]))) / delta_r               # :93
        else:
            delta_r = f32((d_range[1] - d_range[0]) / d_res)                   # :95
            df = (r - f32(d_range[0])) / delta_r                               # :96
    assert tf.dtype == np.float32 and pf.dtype == np.float32 and df.dtype == np.float32
    raw = np.stack([tf, pf, df], axis=1)
    # astype(int) truncates toward zero; NaN (a point on the z axis) is taken as 0, which is where
    # the reference's clamp sends the INT_MIN that an x86 conversion of NaN yields
    def trunc(a):
        return np.where(np.isnan(a), 0.0, np.trunc(np.clip(np.nan_to_num(a, nan=0.0), -2.0 ** 40, 2.0 ** 40))).astype(np.int64)
    theta_idx = np.clip(trunc(tf), 0, v_res - 1)               # :103-106
    phi_idx = np.clip(trunc(pf), 0, h_res - 1)
    dfc = np.where(np.isnan(df), f32(0), df)
    dfc = np.where(dfc < 0, f32(0), dfc)                       # :107 (clamped as a float)
    dfc = np.where(dfc >= d_res, f32(d_res - 1), dfc)          # :108
    depth_idx = dfc.astype(np.int32)                           # :121
    # indexed assignment: the later point of a pixel wins (:114-124)
    feature = np.zeros((1, channel, 1, v_res, h_res), np.float32)
    depth = np.zeros((1, 1, v_res, h_res), np.int32)
    thick = np.zeros((1, v_res, h_res), np.int32)
    for i in range(pts.shape[0]):
        feature[0, :, 0, theta_idx[i], phi_idx[i]] = pts[i]
        depth[0, 0, theta_idx[i], phi_idx[i]] = depth_idx[i]
        thick[0, theta_idx[i], phi_idx[i]] = 1
    bins = np.stack([theta_idx, phi_idx, depth_idx], axis=1).astype(np.int32)
    return feature, depth, thick, bins, raw


# ---- point cloud -> voxels (reference include/point2voxel.h, sphconv/utils/) ---------------

_SYSTEMS = ("spherical", "l-spherical", "cylinder", "l-cylinder", "hybrid", "l-hybrid")


def system_transform(points, coors_range, sphere_coors_range, coord_system):
    """numpy restatement of sphconv/utils/coord_transform.py:8-118 for float32 points:
    -> (system_points [N,4] float32 = (c0, c1, c2, intensity), system_range [6] float64)."""
    pts = np.ascontiguousarray(points, dtype=np.float32)
    x, y, z, intensity = pts[:, 0], pts[:, 1], pts[:, 2], pts[:, 3]
    v, s = coors_range, sphere_coors_range
    with np.errstate(all="ignore"):
        x2y2 = x * x + y * y
        r = np.sqrt(x2y2 + z * z)
        d = np.sqrt(x2y2)
        phi = np.arcsin(y / np.sqrt(x2y2))
        theta = np.arccos(z / r)
        rad = np.radians
        if coord_system == "spherical":        # :8-24
            c = (r, phi, theta); rng = [s[0], rad(s[1]), rad(s[2]), s[3], rad(s[4]), rad(s[5])]
        elif coord_system == "l-spherical":    # :27-42
            c = (np.log(r), phi, theta); rng = [np.log(s[0]), rad(s[1]), rad(s[2]), np.log(s[3]), rad(s[4]), rad(s[5])]
        elif coord_system == "cylinder":       # :45-59
            c = (d, phi, z); rng = [s[0], rad(s[1]), v[2], s[3], rad(s[4]), v[5]]
        elif coord_system == "l-cylinder":     # :62-76
            c = (np.log(d), phi, z); rng = [np.log(s[0]), rad(s[1]), v[2], np.log(s[3]), rad(s[4]), v[5]]
        elif coord_system == "hybrid":         # :79-96
            c = (d, phi, theta); rng = [s[0], rad(s[1]), rad(s[2]), s[3], rad(s[4]), rad(s[5])]
        elif coord_system == "l-hybrid":       # :99-116
            c = (np.log(d), phi, theta); rng = [np.log(s[0]), rad(s[1]), rad(s[2]), np.log(s[3]), rad(s[4]), rad(s[5])]
        else:
            raise ValueError("unknown coord_system %r" % (coord_system,))
    return np.stack([c[0], c[1], c[2], intensity], 1).astype(np.float32), np.array(rng, dtype=np.float64)


def voxel_cells(system_points, system_range, grid_size):
    """Cell of every point as point2voxel.h:436-457 computes it (float32: the pybind11 template is
    instantiated with the points' type, so range and voxel size are float32): (coor [N,3] int64 =
    (idx of c2, idx of c1, idx of c0), valid [N] bool, float bins [N,3] in coordinate order)."""
    f32 = np.float32
    rng = np.asarray(system_range, dtype=np.float64).astype(np.float32)
    g = [int(v) for v in grid_size]
    vs = [f32((rng[3 + i] - rng[i]) / f32(g[i])) for i in range(3)]          # :436-439 (float32 / int -> float32)
    sp = np.asarray(system_points, dtype=np.float32)
    with np.errstate(all="ignore"):
        fb = np.stack([(sp[:, i] - rng[i]) / vs[i] for i in range(3)], axis=1)  # float32
    fl = np.floor(fb)
    ok = np.isfinite(fb).all(1)
    for i in range(3):
        ok &= (fl[:, i] >= 0) & (fl[:, i] < g[i])
    coor = np.where(ok[:, None], np.nan_to_num(fl, nan=0.0, posinf=0.0, neginf=0.0), 0).astype(np.int64)[:, ::-1]
    return coor, ok, fb


def voxelize_cells(points, system_points, coor, valid, max_points, max_voxels, append_mode=0):
    """The sequential loop of points_to_voxel_3d (point2voxel.h:441-505) on given cells: voxels are
    numbered in order of first appearance, keep their first ``max_points`` points, and the loop stops
    at the point that would open voxel number ``max_voxels``.  Returns the reference's dict."""
    pts = np.asarray(points, dtype=np.float32)
    nfeat = pts.shape[1]
    width = nfeat + 3 if append_mode == 1 else nfeat
    voxels = np.zeros((max_voxels, max_points, width), np.float32)
    mask = np.zeros((max_voxels, max_points), np.float32)
    coors = np.zeros((max_voxels, 3), np.int32)
    num = np.zeros((max_voxels,), np.int32)
    table = {}
    voxel_num = 0
    for i in range(pts.shape[0]):
        if not valid[i]:
            continue
        key = (int(coor[i, 0]), int(coor[i, 1]), int(coor[i, 2]))
        vid = table.get(key, -1)
        if vid == -1:
            vid = voxel_num
            if voxel_num >= max_voxels:
                break
            voxel_num += 1
            table[key] = vid
            coors[vid] = key
        n = num[vid]
        if n < max_points:
            mask[vid, n] = 1
            if append_mode == 0:
                voxels[vid, n, :nfeat] = pts[i]
            elif append_mode == 1:
                voxels[vid, n, :nfeat] = pts[i]
                voxels[vid, n, nfeat:nfeat + 3] = system_points[i, :3]
            else:
                voxels[vid, n, :3] = system_points[i, :3]
                voxels[vid, n, 3] = pts[i, 3]
            num[vid] += 1
    return {"voxels": voxels, "coordinates": coors, "num_points_per_voxel": num,
            "voxel_point_mask": mask.reshape(-1, max_points, 1), "voxel_num": voxel_num}


def points_to_voxel_v2(points, coors_range, sphere_coors_range, max_points=1, max_voxels=30000,
                       resolution_HWD=None, coord_system="spherical", append_mode=0):
    """sphconv/utils/voxelize.py:126-214 with a resolution (the transform_funcs branch)."""
    sp, rng = system_transform(points, coors_range, sphere_coors_range, coord_system)
    coor, ok, _ = voxel_cells(sp, rng, resolution_HWD)
    return voxelize_cells(points, sp, coor, ok, max_points, max_voxels, append_mode)


def points_to_voxel_sphere(points, voxel_size, sphere_coors_range, max_points=1, max_voxels=30000):
    """sphconv/utils/voxelize.py:184-206 -> points_to_voxel_3d_sphere_np (include/point2voxel.h:316-399),
    the branch without a resolution: ``voxel_size`` (log r, degrees, degrees) and ``sphere_coors_range``
    (radial bounds in the units of log r, degrees, degrees) -> radians; grid = round(range / voxel size)
    (:337-340); per point theta = acos(z/r), phi = asin(y/sqrt(x^2+y^2)), log r (:349-366), all float32;
    coordinates are (theta, phi, r) bins; then the same sequential loop (:370-392)."""
    f32 = np.float32
    vs = [f32(voxel_size[0]), f32(np.radians(voxel_size[1])), f32(np.radians(voxel_size[2]))]
    s = [float(v) for v in sphere_coors_range]
    rng = np.array([s[0], np.radians(s[1]), np.radians(s[2]), s[3], np.radians(s[4]), np.radians(s[5])]).astype(np.float32)
    grid = [int(np.floor(np.float64(f32(f32(rng[3 + i] - rng[i]) / vs[i])) + 0.5)) for i in range(3)]   # C round()
    pts = np.ascontiguousarray(points, dtype=np.float32)
    x, y, z = pts[:, 0], pts[:, 1], pts[:, 2]
    with np.errstate(all="ignore"):
        x2y2 = x * x + y * y
        r = np.sqrt(x2y2 + z * z)
        theta = np.arccos(z / r)
        phi = np.arcsin(y / np.sqrt(x2y2))
        fb = np.stack([(theta - rng[2]) / vs[2], (phi - rng[1]) / vs[1], (np.log(r) - rng[0]) / vs[0]], axis=1)
    fl = np.floor(fb)
    ok = np.isfinite(fb).all(1)
    for i, g in enumerate((grid[2], grid[1], grid[0])):
        ok &= (fl[:, i] >= 0) & (fl[:, i] < g)
    coor = np.where(ok[:, None], np.nan_to_num(fl, nan=0.0, posinf=0.0, neginf=0.0), 0).astype(np.int64)
    res = voxelize_cells(points, None, coor, ok, max_points, max_voxels, 0)
    res["grid_size"] = grid
    return res


def simple_voxel(voxels, num_points, num_input_features=4):
    """SimpleVoxel.forward (sphconv/vfe.py:222-228): mean of a voxel's points."""
    v = np.asarray(voxels, dtype=np.float32)
    return (v[:, :, :num_input_features].sum(axis=1) / np.asarray(num_points, np.float32).reshape(-1, 1)).astype(np.float32)
