"""Tile / wave / buffer variants beyond the shipping set: the matrix a parity suite runs to show that every
configuration computes the same thing.  ``parity_configs()`` lists them so that a build step can compile them ahead
of time (``prebuilt.build_all(extra=parity_configs())``; nothing is compiled inside a GPU test)."""
from ..arch import MI355X
from . import gfx950_space
from .configs import AttnBwdConfig, AttnConfig, RetBwdConfig, RetConfig

# attention forward, register-fused: (Br, Bc, Nthreads, K buffers, V buffers, waves per SIMD) for every head-size pair below
PARITY_TILES = [
    (128, 64, 256, 2, 2, 2), (128, 64, 256, 1, 1, 2), (128, 64, 256, 2, 1, 1), (128, 64, 256, 1, 2, 1),
    (128, 32, 256, 2, 2, 2), (128, 128, 256, 1, 1, 1), (64, 64, 128, 2, 2, 2), (128, 64, 128, 1, 1, 1),
    (256, 64, 512, 2, 2, 2), (128, 32, 256, 2, 2, 3), (128, 64, 256, 1, 1, 3),
]
PARITY_DIMS = [(64, 64), (128, 128), (64, 128), (256, 256), (192, 192)]
# ... with a kv tile worked through in units (two or more 32-row groups per wave): (Br, Bc, unit rows, Nthreads, waves per SIMD)
UNIT_TILES = [(512, 128, 32, 512, 2), (512, 64, 32, 512, 2), (256, 64, 32, 256, 2), (256, 128, 64, 256, 1), (128, 64, 32, 128, 1)]
UNIT_DIMS = [(64, 64), (128, 128), (64, 128), (128, 64)]


def unit_config(br, bc, unit, nt, wpe, dqk, dv):
    return AttnConfig(br, bc, dqk, dv, dqk, unit, 2, 2, nt, True, waves_per_eu=wpe).set_fuse_type("register")
# attention forward, LDS-fused: (Br, Bc, Nthreads, K bufs, V bufs, W1N, W2N, waves/SIMD)
SHARED_TILES = [(128, 64, 256, 2, 2, 1, 4, 2), (64, 64, 256, 1, 1, 2, 4, 2), (64, 64, 256, 2, 1, 2, 2, 2), (64, 64, 256, 1, 1, 2, 4, 1)]
SHARED_DIMS = [(64, 64), (128, 128), (256, 512)]
# attention backward: head-size pairs run at their defaults, and (Br, Bc, Nthreads, buffers) variants at 128/128
ATTN_BWD_DIMS = [(64, 64), (128, 128), (64, 128), (128, 64), (192, 192), (128, 192), (192, 64), (256, 128), (256, 256), (256, 512)]
ATTN_BWD_TILES = [(64, 32, 128, 2), (64, 64, 128, 2), (128, 64, 256, 3), (128, 32, 256, 2)]
# ... and with one column kernel per output: (Br, Bc, Nthreads, buffers, row waves/SIMD, row Bc, dV waves/SIMD, dK waves/SIMD)
ATTN_BWD_SPLIT_TILES = [(128, 32, 256, 2, 2, 32, 2, 2), (128, 64, 256, 2, 2, 32, 2, 1), (128, 32, 256, 3, 2, 32, 3, 2),
                        (64, 32, 128, 2, 1, 32, 1, 1)]


def attn_bwd_split_config(br, bc, nt, st, row_wpe, row_bc, dv_wpe, dk_wpe, dqk=128, dv=128):
    return AttnBwdConfig(br, bc, dqk, dv, nt, st, waves_per_eu=1, row_waves_per_eu=row_wpe, row_Bc=row_bc, col_split=1,
                         dv_waves_per_eu=dv_wpe, dk_waves_per_eu=dk_wpe)
# kv-splitting variants: (d_qk, d_v, splits)
SPLIT_VARIANTS = [(128, 128, 4), (128, 128, 8), (64, 64, 2)]
# register-fused configurations the stand-alone attention benchmark times (csrc/benchmarks/attention.hip): (d, Br, Bc, threads, waves/SIMD)
STANDALONE_BENCH_TILES = [(64, 128, 64, 256, 2), (64, 128, 32, 256, 2), (64, 64, 64, 128, 2), (128, 256, 64, 512, 3),
                          (128, 256, 64, 512, 2), (128, 128, 64, 256, 3), (128, 128, 32, 256, 3)]


def persistent_graph_config():
    """A 256-row, 512-thread attention configuration with one row group per wave: takes the persistent-block kernel on
    short rows (the graph-capture test of that kernel runs it)."""
    return AttnConfig(256, 128, 128, 128, 128, 128, 2, 2, 512, True, waves_per_eu=2).set_fuse_type("register")


def ret_register_wide():
    """The register-fused RetNet forward at d_qk 256, d_v 512 (the reference has this variant,
    csrc/kernels/retnet/regfuse/regfuse.h:267-340): 256 output accumulators per lane."""
    return RetConfig(128, 64, 256, 512, 256, 64, 1, 1, 1, 256, True, waves_per_eu=1).set_fuse_type("register")


def ret_register_wide_buffered():
    """The same kernel with a second buffer per stream: two K / mask buffers next to one V buffer on 64-row tiles, and every
    stream double-buffered on 32-row tiles (one barrier per tile).  The run-time buffer parity and the copies threaded
    between the matrix steps take other paths here than in the single-buffer build."""
    return [RetConfig(128, 64, 256, 512, 256, 64, 2, 2, 1, 256, True, waves_per_eu=1).set_fuse_type("register"),
            RetConfig(128, 32, 256, 512, 256, 32, 2, 2, 2, 256, True, waves_per_eu=1).set_fuse_type("register")]


def ret_shared_wide_one_wave():
    """The LDS-fused RetNet forward with four waves at d_v 512: a wave of the second grid holds 32 rows x 512 columns, the
    same 256 accumulation registers per lane, and rescales them in place like the register-fused kernel."""
    cfg = RetConfig(128, 64, 256, 512, 256, 64, 1, 1, 1, 256, True, 1, 4, waves_per_eu=1)
    cfg.fuse_type = "shared"
    return cfg


# RetNet backward with dS stored by the dQ pass and read back by a dK kernel of its own: (d_qk, d_v, Br, Bc, threads, kv rows of the dK kernel)
RET_BWD_STORED_DS = [(256, 512, 128, 64, 256, 128), (256, 512, 128, 64, 256, 256), (256, 512, 128, 32, 256, 256), (64, 128, 64, 32, 128, 128)]


# ... and with two or three Y/mask buffers and one or two Z buffers: the dS stores then stay in flight across tile
# boundaries next to the ring's copies, under different wait counts (last element: (Y buffers, Z buffers))
RET_BWD_STORED_DS_STAGED = [(256, 512, 128, 32, 256, 128, (2, 2)), (256, 512, 128, 32, 256, 256, (2, 1)),
                            (64, 128, 64, 32, 128, 128, (3, 2)), (128, 128, 128, 32, 256, 128, (3, 2)), (256, 256, 128, 32, 256, 128, (3, 2))]


def ret_bwd_stored_ds_config(dqk, dv, br, bc, nt, ds_rows, stages=(1, 1)):
    n = nt // 64
    return RetBwdConfig(br, bc, dqk, dv, n, n, n, n, nt, True, BlockKSmem=dqk, num_stages_qk=stages[0], num_stages_mask=stages[0],
                        num_stages_dv=stages[1], num_stages_ds=stages[0], num_stages_dq=stages[1], waves_per_eu=1, ds_rows=ds_rows)


def parity_configs(arch=None):
    arch = arch or MI355X()
    out = []
    for d, br, bc, nt, wpe in STANDALONE_BENCH_TILES:
        out.append(AttnConfig(br, bc, d, d, d, bc, 2, 2, nt, True, waves_per_eu=wpe).set_fuse_type("register"))
    # RetNet forward variants at 128/128 (register and both wave grids of the LDS-fused kernel)
    for fuse, extra in (("register", {}), ("shared", dict(warps_mma1_n=1, warps_mma_n=4)), ("shared", dict(warps_mma1_n=2, warps_mma_n=2))):
        for st in ((1, 1), (2, 2)):
            cfg = RetConfig(128 if fuse == "register" else 64, 64, 128, 128, 128, 64, st[0], st[0], st[1], 256, True, waves_per_eu=1, **extra)
            cfg.fuse_type = fuse
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
    out.append(persistent_graph_config())
    out.append(ret_register_wide())
    out += ret_register_wide_buffered()
    out.append(ret_shared_wide_one_wave())
    for t in RET_BWD_STORED_DS:
        out += [ret_bwd_stored_ds_config(*t), ret_bwd_stored_ds_config(*t[:5], 0)]      # and the same passes without it
    for t in RET_BWD_STORED_DS_STAGED:
        out += [ret_bwd_stored_ds_config(*t[:6], stages=t[6]), ret_bwd_stored_ds_config(*t[:5], 0, stages=t[6])]
    out += [attn_bwd_split_config(*t) for t in ATTN_BWD_SPLIT_TILES]
    out.append(AttnBwdConfig(64, 64, 128, 128, 128, 2, row_waves_per_eu=2, row_Bc=32))      # row kernel with a tile height of its own
    for br, bc, nt, st in ATTN_BWD_TILES:
        for row_wpe in (1, 2):
            cfg = AttnBwdConfig(br, bc, 128, 128, nt, st, row_waves_per_eu=row_wpe)
            if gfx950_space.attn_backward_valid(cfg, arch):
                out.append(cfg)
    for dqk, dv in PARITY_DIMS:
        for br, bc, nt, sq, sv, wpe in PARITY_TILES:
            cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, waves_per_eu=wpe).set_fuse_type("register")
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
            if (sq, sv) == (2, 2):
                piped = AttnConfig(br, bc, dqk, dv, dqk, bc, 2, 2, nt, True, waves_per_eu=wpe, sw_pipeline=1).set_fuse_type("register")
                if gfx950_space.forward_valid(piped, arch):
                    out.append(piped)
    for dqk, dv in UNIT_DIMS:
        for t in UNIT_TILES:
            cfg = unit_config(*t, dqk, dv)
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
    for dqk, dv, ns in SPLIT_VARIANTS:
        out.append(AttnConfig(128, 64, dqk, dv, dqk, 64, 2, 2, 256, True, waves_per_eu=2, kv_splits=ns).set_fuse_type("register"))
    for dqk, dv in SHARED_DIMS:
        for br, bc, nt, sq, sv, w1n, w2n, wpe in SHARED_TILES:
            cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, w1n, w2n, waves_per_eu=wpe)
            cfg.fuse_type = "shared"
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
    return out
