"""Search space and validity model for MI355X (gfx950).

The knobs that matter on CDNA4 are not the ones that matter on Ampere: tiles are built from
32x32x16 MFMAs so every wave owns whole 32-row groups; K/V reach LDS by LDS-DMA so "stages" are
whole-tile buffers; and the register file is split between the resident waves of a SIMD, so the
occupancy target (``waves_per_eu``) is itself a knob.  Validity is LDS bytes (160 KB per CU, shared by
all resident blocks) and a per-lane register estimate (512 / waves_per_eu).
"""
from .configs import AttnConfig, RetConfig, RetBwdConfig, AttnBwdConfig


class NoValidConfigError(ValueError):
    """No configuration of the gfx950 space fits the problem (head sizes beyond what one wave's registers or
    the LDS hold, a sequence length no tile divides)."""

WAVE = 64
MFMA_M = 32
BR_LIST = (64, 128, 256, 512)
BC_LIST = (32, 64, 128)
THREADS = (128, 256, 512)
STAGES = ((1, 1), (2, 2), (2, 1), (1, 2))
KV_SPLITS = (2, 4, 8, 16)


def _waves(cfg):
    return cfg.Nthreads // WAVE


def rows_per_wave(cfg):
    return cfg.Br // _waves(cfg)


def blocks_per_cu(cfg):
    """Resident blocks per CU implied by the occupancy target (4 SIMDs per CU)."""
    return max(1, (cfg.waves_per_eu * 4) // _waves(cfg))


def unit_rows(cfg):
    """kv rows of one scores -> softmax -> PV unit of the register-fused attention forward (plain schedule):
    ``BlockKSmem2``, a divisor of Bc; the whole tile everywhere else."""
    if cfg.operation == "attn" and cfg.fuse_type == "register" and not getattr(cfg, "sw_pipeline", 0):
        return getattr(cfg, "BlockKSmem2", cfg.Bc) or cfg.Bc
    return cfg.Bc


def dma_divisible(cfg):
    nt = cfg.Nthreads
    return (cfg.Bc * cfg.Kd // 8) % nt == 0 and (cfg.Bc * cfg.D // 8) % nt == 0


# ---- forward (attention and RetNet) ------------------------------------------------------------------
def forward_lds_bytes(cfg):
    main = cfg.num_stages_qk * cfg.Bc * cfg.Kd * 2 + cfg.num_stages_v * cfg.Bc * cfg.D * 2
    if cfg.operation == "ret":
        main += max(cfg.num_stages_mask, cfg.num_stages_qk) * cfg.Br * cfg.Bc * 2
    if cfg.fuse_type == "shared":
        main += cfg.Br * (cfg.Bc * 2 + 16)            # P tile, fp16, padded rows
        main += (cfg.warps_mma1_n * cfg.Br + cfg.Br) * 4 + 64
        return max(main, cfg.Br * (cfg.D * 2 + 16 * cfg.warps_mma_n))
    epilogue = cfg.Br * (cfg.D * 2 + 16)
    return max(main, epilogue)


def forward_reg_estimate(cfg):
    """Per-lane 32-bit registers of the dominant live set."""
    if cfg.fuse_type == "shared":
        nw = _waves(cfg)
        rt1 = cfg.Br // (nw // cfg.warps_mma1_n) // 32
        nt1 = cfg.Bc // cfg.warps_mma1_n // 32
        o_regs = cfg.Br * cfg.D // (nw * 64)
        return rt1 * (cfg.Kd // 16) * 4 + rt1 * nt1 * 16 + o_regs + 48
    rt = rows_per_wave(cfg) // MFMA_M
    unit = unit_rows(cfg)
    q_regs = rt * (cfg.Kd // 16) * 4
    s_regs = rt * (unit // 32) * 16
    p_regs = rt * (unit // 32) * 4              # fp16 P, built while the fp32 scores retire
    if cfg.fuse_type == "register":
        o_regs = rt * (cfg.D // 32) * 16
    else:
        # shared fuse: the waves split D between them for the second contraction
        o_regs = (cfg.Br // MFMA_M) * (cfg.D // 32) * 16 // _waves(cfg)
    if getattr(cfg, "sw_pipeline", 0):
        s_regs *= 2                                   # current and next score tile are both live
    # a count of what must be live, not a prediction of what the register allocator achieves: candidates that
    # pass it and still spill are rejected by the tuning loop from the compiler's own resource report
    # (a kernel this close to its budget derives its operand addresses from one register each and keeps two-slot
    # operand rings: 24 registers besides the tiles)
    return q_regs + s_regs + p_regs + o_regs + (24 if unit < cfg.Bc else 32)


def forward_likely_spills(cfg):
    """Register-fused configurations whose accumulator alone takes half of a wave's budget have always come
    back from hipcc with hundreds of bytes of scratch.  The tuning loop lets the compiler's report decide;
    the untuned defaults stay clear of them without compiling anything."""
    if cfg.fuse_type != "register":
        return False
    rt = rows_per_wave(cfg) // MFMA_M
    o_regs = rt * (cfg.D // 32) * 16
    return o_regs > 128 and rt * (cfg.Kd // 16) * 4 + rt * (cfg.Bc // 32) * 16 + o_regs > 320


def shared_grid_ok(cfg):
    """Wave grids of the LDS-fused kernels: W1M x W1N over (rows, kv), W2M x W2N over (rows, d)."""
    nw, w1n, w2n = _waves(cfg), cfg.warps_mma1_n, cfg.warps_mma_n
    if not w1n or not w2n or nw % w1n or nw % w2n:
        return False
    w1m, w2m = nw // w1n, nw // w2n
    if cfg.Br % (32 * w1m) or cfg.Bc % (32 * w1n) or cfg.Br % (32 * w2m) or cfg.D % (32 * w2n):
        return False
    return True


def forward_valid(cfg, arch):
    if cfg.fuse_type == "shared":
        if cfg.Nthreads % WAVE or not shared_grid_ok(cfg):
            return False
    elif cfg.Nthreads % WAVE or cfg.Br % (MFMA_M * _waves(cfg)):
        return False
    if cfg.Bc % 32 or cfg.Kd % 64 or cfg.D % 64:
        return False
    unit = unit_rows(cfg)
    if unit % 32 or cfg.Bc % unit:
        return False
    if unit < cfg.Bc and not (cfg.num_stages_qk == 2 and cfg.num_stages_v == 2):   # no barrier between the contractions of a unit
        return False
    if _waves(cfg) > 4 * cfg.waves_per_eu:           # the block itself needs that many waves per SIMD
        return False
    if not dma_divisible(cfg):
        return False
    if getattr(cfg, "sw_pipeline", 0):
        # needs 2+2 buffers and K copies made of whole 32-row units
        rows_per_dma = cfg.Nthreads * 8 // cfg.Kd if (cfg.Nthreads * 8) % cfg.Kd == 0 else 0
        if not (cfg.num_stages_qk == 2 and cfg.num_stages_v == 2 and cfg.fuse_type == "register"):
            return False
        if rows_per_dma == 0 or rows_per_dma > 32 or 32 % rows_per_dma:
            return False
    if forward_lds_bytes(cfg) * blocks_per_cu(cfg) > arch.smem_cap:
        return False
    return forward_reg_estimate(cfg) <= arch.register_per_thread // cfg.waves_per_eu




def forward_candidates(op, br, bc, dim_qk, dim_v, fuse_types=("register", "shared"), with_splits=False):
    out = []
    for nthreads in THREADS:
        for st_qk, st_v in STAGES:
            for wpe in (1, 2, 3):
                for fuse in fuse_types:
                    if fuse == "shared":
                        if st_qk == st_v and wpe <= 2:   # the LDS-fused kernels gain little from mixed buffering
                            out.extend(_shared_candidates(op, br, bc, dim_qk, dim_v, st_qk, st_v, nthreads, wpe))
                        continue
                    if op == "attn":
                        cfg = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, bc, st_qk, st_v, nthreads, True, waves_per_eu=wpe)
                    else:
                        cfg = RetConfig(br, bc, dim_qk, dim_v, dim_qk, bc, st_qk, st_qk, st_v, nthreads, True, waves_per_eu=wpe)
                    out.append(cfg.set_fuse_type(fuse))
                    if op == "attn" and fuse == "register" and (st_qk, st_v) == (2, 2):
                        piped = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, bc, 2, 2, nthreads, True, waves_per_eu=wpe, sw_pipeline=1)
                        out.append(piped.set_fuse_type(fuse))
                    if op == "attn" and fuse == "register" and (st_qk, st_v) == (2, 2) and br // (nthreads // WAVE) >= 2 * MFMA_M:
                        # two or more 32-row groups per wave: a kv tile worked through in 32-row units keeps one
                        # small score tile live, which is what lets such a wave share its SIMD with a second one
                        for unit in (32, 64):
                            if unit < bc:
                                for ns in (1,) + (KV_SPLITS if with_splits else ()):
                                    u = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, unit, 2, 2, nthreads, True, waves_per_eu=wpe, kv_splits=ns)
                                    out.append(u.set_fuse_type(fuse))
                    if op == "attn" and fuse == "register" and with_splits and st_qk == st_v:
                        for ns in KV_SPLITS:   # long kv, few query rows: cut the kv range so every CU gets work
                            sp = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, bc, st_qk, st_v, nthreads, True, waves_per_eu=wpe, kv_splits=ns)
                            out.append(sp.set_fuse_type(fuse))
    return out


def _shared_candidates(op, br, bc, dim_qk, dim_v, st_qk, st_v, nthreads, wpe):
    out = []
    nw = nthreads // WAVE
    for w1n in (1, 2, 4):
        for w2n in sorted({nw, max(1, nw // 2), max(1, nw // 4)}):
            if op == "attn":
                cfg = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, bc, st_qk, st_v, nthreads, True, w1n, w2n, waves_per_eu=wpe)
            else:
                cfg = RetConfig(br, bc, dim_qk, dim_v, dim_qk, bc, st_qk, st_qk, st_v, nthreads, True, w1n, w2n, waves_per_eu=wpe)
            cfg.fuse_type = "shared"
            if shared_grid_ok(cfg):
                out.append(cfg)
    return out


def default_forward_config(op, dim_qk, dim_v, arch, seq_q=None, seq_k=None):
    """A configuration that is valid for every supported head size; used before/without tuning."""
    prefs = [(256, 64, 512, 2, 2, 2), (128, 64, 256, 2, 2, 2), (128, 64, 256, 1, 1, 2), (128, 64, 256, 1, 1, 1), (128, 32, 256, 1, 1, 1),
             (64, 32, 128, 1, 1, 1)]
    if op == "ret" and dim_v == 512 and not ((seq_q and seq_q % 128) or (seq_k and seq_k % 64)):
        # 32 rows x 512 columns per wave fill the 256 accumulation registers of a wave that has its SIMD to itself;
        # the RetNet kernel is written so that this builds without scratch, and at d_qk 256 it leads every mask mode
        cfg = RetConfig(128, 64, dim_qk, dim_v, dim_qk, 64, 1, 1, 1, 256, True, waves_per_eu=1)
        cfg.set_fuse_type("register")
        if forward_valid(cfg, arch):
            return cfg
    for br, bc, nt, sq, sv, wpe in prefs:
        if (seq_q and seq_q % br) or (seq_k and seq_k % bc):
            continue
        if op == "attn":
            cfg = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, bc, sq, sv, nt, True, waves_per_eu=wpe)
        else:
            cfg = RetConfig(br, bc, dim_qk, dim_v, dim_qk, bc, sq, sq, sv, nt, True, waves_per_eu=wpe)
        cfg.set_fuse_type("register")
        if forward_valid(cfg, arch) and not forward_likely_spills(cfg):
            return cfg
    # wide value heads: the LDS-fused kernel keeps the accumulator at Br*D/(64*waves) registers
    for br, bc, nt, w1n, w2n in ((128, 64, 512, 2, 8), (64, 64, 256, 2, 4)):
        if (seq_q and seq_q % br) or (seq_k and seq_k % bc):
            continue
        if op == "attn":
            cfg = AttnConfig(br, bc, dim_qk, dim_v, dim_qk, bc, 1, 1, nt, True, w1n, w2n, waves_per_eu=nt // 256)
        else:
            cfg = RetConfig(br, bc, dim_qk, dim_v, dim_qk, bc, 1, 1, 1, nt, True, w1n, w2n, waves_per_eu=nt // 256)
        cfg.fuse_type = "shared"
        if forward_valid(cfg, arch):
            return cfg
    raise NoValidConfigError(f"no default {op} configuration fits dim_qk={dim_qk} dim_v={dim_v} seq=({seq_q},{seq_k})")


# ---- backward (RetNet) ---------------------------------------------------------------------------------
# Three passes of one chained-contraction kernel (dV, dK, dQ).  Br = block-resident rows, Bc = streamed rows
# per step, for every pass; both sequence lengths must divide by both.
BWD_BR_LIST = (64, 128, 256, 512)
BWD_BC_LIST = (32, 64)


def backward_dv_cols(cfg):
    """dV columns one block produces.  With one wave per SIMD the output accumulators live in the 256
    accumulation registers, which hold a 32-row group of up to 512 columns; otherwise (or for wider
    values) the pass is sliced into 256-column blocks over grid.y and repeats its first contraction."""
    rt = cfg.Br // _waves(cfg) // MFMA_M
    if cfg.waves_per_eu == 1 and rt * cfg.D <= 512:
        return cfg.D
    return min(cfg.D, 256)


def _backward_passes(cfg):
    """(first-contraction width, output columns per block, buffers of the first stream, of the second) of the dV, dK
    and dQ passes."""
    return ((cfg.Kd, backward_dv_cols(cfg), cfg.num_stages_qk, cfg.num_stages_dv),
            (cfg.D, cfg.Kd, cfg.num_stages_ds, cfg.num_stages_dq), (cfg.D, cfg.Kd, cfg.num_stages_ds, cfg.num_stages_dq))


def backward_lds_bytes(cfg):
    worst = 0
    for kx, dzb, sy, sz in _backward_passes(cfg):
        main = sy * (cfg.Bc * kx * 2 + cfg.Br * cfg.Bc * 2) + sz * cfg.Bc * dzb * 2
        worst = max(worst, main, cfg.Br * (dzb * 2 + 16))
    return worst


def backward_reg_estimate(cfg):
    """(vector registers, accumulation registers) of the hungriest pass."""
    rt = cfg.Br // _waves(cfg) // MFMA_M
    vec = acc = 0
    for kx, dzb, _, _ in _backward_passes(cfg):
        vec = max(vec, rt * (kx // 16) * 4 + rt * (cfg.Bc // 32) * 24 + 64)
        acc = max(acc, rt * (dzb // 32) * 16)
    return vec, acc


DS_ROWS = (128, 256)          # kv rows per block of the dK kernel that reads a stored dS (64-row query tiles, two stages)
DS_TILE = 64


def backward_valid(cfg, arch):
    nw = _waves(cfg)
    ds_rows = getattr(cfg, "ds_rows", 0)
    if ds_rows:
        if ds_rows not in DS_ROWS or cfg.Br % DS_TILE or cfg.waves_per_eu != 1:
            return False
        # the row pass stages a dS tile behind its stream buffers; the dK kernel holds two (Q tile, dS tile) pairs
        row_lds = cfg.num_stages_ds * (cfg.Bc * cfg.D * 2 + cfg.Br * cfg.Bc * 2) + cfg.num_stages_dq * cfg.Bc * cfg.Kd * 2
        if row_lds + cfg.Br * (cfg.Bc * 2 + 16) > arch.smem_cap:
            return False
        if 2 * DS_TILE * (cfg.Kd + ds_rows) * 2 > arch.smem_cap:
            return False
    if cfg.Nthreads % WAVE or cfg.Br % (MFMA_M * nw) or cfg.Bc % 32:
        return False
    if nw > 4 * cfg.waves_per_eu:
        return False
    for sy, sz in ((cfg.num_stages_qk, cfg.num_stages_dv), (cfg.num_stages_ds, cfg.num_stages_dq)):
        if sy not in (1, 2, 3) or sz not in (1, 2):
            return False
        if sy == 3 and sz != 2:      # the three-buffer schedule prefetches Z one tile ahead
            return False
    if cfg.num_stages_mask != cfg.num_stages_qk:               # the mask tile travels with the first stream
        return False
    nt = cfg.Nthreads
    for cols in (cfg.Kd, cfg.D, backward_dv_cols(cfg), cfg.Br):   # every streamed tile must split evenly over the threads
        if (cfg.Bc * cols // 8) % nt:
            return False
    if (cfg.Br * cfg.Bc // 8) % nt:
        return False
    if backward_lds_bytes(cfg) * blocks_per_cu(cfg) > arch.smem_cap:
        return False
    vec, acc = backward_reg_estimate(cfg)
    if cfg.waves_per_eu == 1:          # 256 vector + 256 accumulation registers
        return vec <= 256 and acc <= 256
    return vec + acc <= arch.register_per_thread // cfg.waves_per_eu


BWD_STAGES = ((1, 1), (2, 2), (2, 1), (3, 2))       # (buffers of the first stream, of the second) of a pass


def backward_candidates(br, bc, dim_qk, dim_v):
    """Every combination of buffer counts for the dV pass and for the d_v-contracting passes: where d_v differs from
    d_qk the two kinds of pass stream tiles of different widths and the best counts differ with them."""
    out = []
    for nthreads in (128, 256, 512):
        for st_y, st_z in BWD_STAGES:
            for st_ds, st_dq in (BWD_STAGES if dim_qk != dim_v else ((st_y, st_z),)):
                for wpe in (1, 2):
                    n = nthreads // WAVE
                    kw = dict(BlockKSmem=dim_qk, num_stages_qk=st_y, num_stages_mask=st_y, num_stages_dv=st_z,
                              num_stages_ds=st_ds, num_stages_dq=st_dq, waves_per_eu=wpe)
                    out.append(RetBwdConfig(br, bc, dim_qk, dim_v, n, n, n, n, nthreads, True, **kw))
                    if wpe == 1:          # ... and with dS stored by the dQ pass for a dK kernel of its own (needs the workspace)
                        for ds_rows in DS_ROWS:
                            out.append(RetBwdConfig(br, bc, dim_qk, dim_v, n, n, n, n, nthreads, True, ds_rows=ds_rows, **kw))
    return out


def default_backward_config(dim_qk, dim_v, arch, seq_q=None, seq_k=None):
    prefs = ((128, 32, 256, 3, 2, 1), (128, 32, 256, 2, 2, 1), (64, 32, 128, 2, 2, 1), (64, 32, 128, 1, 1, 1), (64, 32, 128, 1, 1, 2),
             (64, 64, 128, 1, 1, 1))
    if dim_v == 512:            # measured at d_qk 256: 64-row streamed tiles with single buffers lead the three-buffer ring of 32-row tiles
        prefs = ((128, 64, 256, 1, 1, 1),) + prefs
    for br, bc, nt, sy, sz, wpe in prefs:
        if any(s and (s % br or s % bc) for s in (seq_q, seq_k)):
            continue
        n = nt // WAVE
        cfg = RetBwdConfig(br, bc, dim_qk, dim_v, n, n, n, n, nt, True, BlockKSmem=dim_qk, num_stages_qk=sy,
                           num_stages_mask=sy, num_stages_dv=sz, num_stages_ds=sy, num_stages_dq=sz, waves_per_eu=wpe)
        if backward_valid(cfg, arch):
            return cfg
    raise NoValidConfigError(f"no default ret_bwd configuration fits dim_qk={dim_qk} dim_v={dim_v} seq=({seq_q},{seq_k})")


# ---- backward (attention) ------------------------------------------------------------------------------
# A column kernel (dV, dK) and a row kernel (dQ) share Br (resident rows) and Bc (streamed rows per step).
ATTN_BWD_BR_LIST = (64, 128, 256, 512)
ATTN_BWD_BC_LIST = (32, 64)


def attn_backward_lds_bytes(cfg):
    stage = cfg.Bc * (cfg.Kd + cfg.D) * 2 + 1024            # streamed tile pair + per-row statistics slot
    return max(cfg.num_stages_qk * stage, cfg.Br * (max(cfg.Kd, cfg.D) * 2 + 16))


def attn_backward_reg_estimate(cfg):
    """(vector registers, accumulation registers) of the column kernel, the hungrier of the two."""
    rt = cfg.Br // _waves(cfg) // MFMA_M
    nt = cfg.Bc // 32
    vec = rt * ((cfg.Kd + cfg.D) // 16) * 4 + rt * nt * 16 + 72
    acc = rt * ((cfg.Kd + cfg.D) // 32) * 16                # dV + dK accumulators
    scores = rt * nt * 32                                    # S and dP tiles
    if cfg.waves_per_eu == 1 and acc + scores > 256:        # the kernel then keeps the score tiles in vector registers
        return vec + scores - rt * nt * 16, acc
    return vec, acc + scores


def attn_backward_split_reg_estimates(cfg):
    """(dV-only column kernel, dK-only column kernel) registers per lane: resident fragments, the output
    accumulators, the score tiles, the fp16 operand of the second contraction, addresses."""
    rt = cfg.Br // _waves(cfg) // MFMA_M
    nt = cfg.Bc // 32
    dv = rt * (cfg.Kd // 16) * 4 + rt * (cfg.D // 32) * 16 + rt * nt * 16 + rt * nt * 8 + 48
    dk = rt * ((cfg.Kd + cfg.D) // 16) * 4 + rt * (cfg.Kd // 32) * 16 + rt * nt * 32 + rt * nt * 8 + 48
    return dv, dk


def _one_wave_fits(rt, frag_cols, out_cols, score_tiles):
    """One wave per SIMD: 256 vector + 256 accumulation registers.  Resident fragments, the fp16 operand and
    addresses are vector registers; outputs are accumulation registers and the score tiles join them if there
    is room, else they are vector registers too."""
    vec = rt * (frag_cols // 16) * 4 + rt * 8 + 48
    acc = rt * (out_cols // 32) * 16
    scores = rt * score_tiles * 16
    if acc + scores <= 256:
        return vec <= 256 and acc <= 256
    return vec + scores <= 256 and acc <= 256


def _split_budget_ok(regs, rt, frag_cols, out_cols, score_tiles, wpe, nw, lds_bytes, arch):
    """One half of a split column kernel at ``wpe`` waves per SIMD."""
    if wpe not in (1, 2, 3) or nw > 4 * wpe:
        return False
    if lds_bytes * (max(1, (wpe * 4) // nw) if wpe > 1 else 1) > arch.smem_cap:
        return False
    if wpe == 1:
        return _one_wave_fits(rt, frag_cols, out_cols, score_tiles)
    return regs <= arch.register_per_thread // wpe


def attn_backward_valid(cfg, arch):
    nw = _waves(cfg)
    if cfg.Nthreads % WAVE or cfg.Br % (MFMA_M * nw) or cfg.Bc % 32 or cfg.Bc > 128:
        return False
    if nw > 4 * cfg.waves_per_eu or cfg.num_stages_qk not in (2, 3):
        return False
    for cols in (cfg.Kd, cfg.D):
        if cols % 64:                                              # the dual swizzle covers every multiple of 64
            return False
        if (cfg.Bc * cols // 8) % cfg.Nthreads:
            return False
    # an occupancy target above one wave per SIMD must be reachable; at one wave per SIMD a single block per CU will do
    if attn_backward_lds_bytes(cfg) * (blocks_per_cu(cfg) if cfg.waves_per_eu > 1 else 1) > arch.smem_cap:
        return False
    row_wpe = getattr(cfg, "row_waves_per_eu", cfg.waves_per_eu)
    row_bc = getattr(cfg, "row_Bc", cfg.Bc)
    if row_bc != cfg.Bc:                                     # a tile height of its own only with a budget of its own
        if row_wpe == cfg.waves_per_eu or row_bc % 32 or row_bc > 128:
            return False
        if any((row_bc * cols // 8) % cfg.Nthreads for cols in (cfg.Kd, cfg.D)):
            return False
    if row_wpe != cfg.waves_per_eu:
        if cfg.waves_per_eu != 1 or row_wpe != 2 or nw > 8:
            return False
        if attn_backward_row_reg_estimate(cfg) > arch.register_per_thread // 2:
            return False
        row_lds = max(cfg.num_stages_qk * row_bc * (cfg.Kd + cfg.D) * 2, cfg.Br * (cfg.Kd * 2 + 16))
        if row_lds * max(1, 8 // nw) > arch.smem_cap:
            return False
    elif cfg.waves_per_eu == 1:                              # the row kernel on the column kernel's budget
        if not _one_wave_fits(cfg.Br // nw // MFMA_M, cfg.Kd + cfg.D, cfg.Kd, 2 * (row_bc // 32)):
            return False
    if getattr(cfg, "col_split", 0):
        rt = cfg.Br // nw // MFMA_M
        dv, dk = attn_backward_split_reg_estimates(cfg)
        lds = attn_backward_lds_bytes(cfg)
        return (cfg.waves_per_eu == 1 and
                _split_budget_ok(dv, rt, cfg.Kd, cfg.D, cfg.Bc // 32, cfg.dv_waves_per_eu, nw, lds, arch) and
                _split_budget_ok(dk, rt, cfg.Kd + cfg.D, cfg.Kd, 2 * (cfg.Bc // 32), cfg.dk_waves_per_eu, nw, lds, arch))
    vec, acc = attn_backward_reg_estimate(cfg)
    if cfg.waves_per_eu == 1:
        return vec <= 256 and acc <= 256
    return vec + acc <= arch.register_per_thread // cfg.waves_per_eu


def attn_backward_row_reg_estimate(cfg):
    """Registers of the row kernel (resident Q and dO fragments, the dQ accumulators, S and dP, the fp16
    operand of the second contraction, addresses): 206 measured at 128/128 with 32-row tiles, 238 with 64."""
    rt = cfg.Br // _waves(cfg) // MFMA_M
    nt = getattr(cfg, "row_Bc", cfg.Bc) // 32
    return rt * ((cfg.Kd + cfg.D) // 16) * 4 + rt * (cfg.Kd // 32) * 16 + rt * nt * 32 + rt * nt * 8 + 48


def attn_backward_candidates(br, bc, dim_qk, dim_v):
    out = []
    for nthreads in (128, 256, 512):
        for stages in (2, 3):
            for wpe in (1, 2):
                out.append(AttnBwdConfig(br, bc, dim_qk, dim_v, nthreads, stages, waves_per_eu=wpe))
            for row_bc in (32, 64):
                out.append(AttnBwdConfig(br, bc, dim_qk, dim_v, nthreads, stages, waves_per_eu=1, row_waves_per_eu=2, row_Bc=row_bc))
            # one column kernel per output, each on the largest occupancy it fits
            for row_wpe in (1, 2):
                for dv_wpe, dk_wpe in ((3, 2), (2, 2), (2, 1), (1, 1)):
                    out.append(AttnBwdConfig(br, bc, dim_qk, dim_v, nthreads, stages, waves_per_eu=1, row_waves_per_eu=row_wpe,
                                             col_split=1, dv_waves_per_eu=dv_wpe, dk_waves_per_eu=dk_wpe))
    return out


def default_attn_backward_config(dim_qk, dim_v, arch, seq_q=None, seq_k=None):
    for br, bc, nt, st, wpe in ((128, 32, 256, 3, 1), (128, 32, 256, 2, 1), (64, 32, 128, 3, 1), (64, 32, 128, 2, 1), (64, 32, 128, 2, 2)):
        if any(s and (s % br or s % bc) for s in (seq_q, seq_k)):
            continue
        for row_wpe in ((2, wpe) if wpe == 1 else (wpe,)):            # the row kernel at two waves per SIMD where it fits
            cfg = AttnBwdConfig(br, bc, dim_qk, dim_v, nt, st, waves_per_eu=wpe, row_waves_per_eu=row_wpe)
            if attn_backward_valid(cfg, arch):
                return cfg
    # head sizes whose dV and dK accumulators cannot share a wave: one column kernel per output
    for br, bc, nt, st in ((128, 32, 256, 3), (128, 32, 256, 2), (64, 32, 128, 2)):
        if any(s and (s % br or s % bc) for s in (seq_q, seq_k)):
            continue
        cfg = AttnBwdConfig(br, bc, dim_qk, dim_v, nt, st, waves_per_eu=1, col_split=1)
        if attn_backward_valid(cfg, arch):
            return cfg
    raise NoValidConfigError(f"no default attn_bwd configuration fits dim_qk={dim_qk} dim_v={dim_v} seq=({seq_q},{seq_k})")
