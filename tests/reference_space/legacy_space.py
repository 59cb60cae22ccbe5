"""Search space and validity model of the reference for NVIDIA parts (A100 / RTX 4090).

Nothing here is compiled or run on MI355X.  It is kept, restated, because the reference ships its
tuning logs (docs/tuning_result_*/profile_result_*.txt) and the ordered list of configurations in
those logs is the only known-answer data for the tuner: tests/test_enumeration.py checks that this
module reproduces them line by line.

Rules restated from reference python/autotuner/tunner.py:13-225 (``generate_configs``,
``validate_register_fuse``, ``validate_shared_fuse``, ``validate_kernel``).
"""
from attention_autotuner_amd.autotuner.configs import AttnConfig, RetConfig, RetBwdConfig, balanced_wave_split

_THREADS = (128, 256)


def _qk_slabs(dim_qk):
    """(BlockKSmem, num_stages_qk) candidates: whole head dim single-staged, or a pipelined slab."""
    half = dim_qk / 2
    slab = 64 if half > 64 else 32 if half > 32 else 16
    return [(dim_qk, 1), (slab, 2)]


def _v_slabs(bc):
    return [(bc, 1), (bc // 4, 2)]


def _thread_rule_ok(br, bc, slab_qk, slab_v, nthreads):
    """256-thread variants the reference's copy atoms cannot serve."""
    if nthreads != 256:
        return True
    if br == 32 and bc == 32:
        return False
    if slab_qk == 32 and slab_v == 32:
        return False
    if (br == 32 or bc == 32) and slab_qk == 32:
        return False
    return True


def forward_candidates(op, br, bc, dim_qk, dim_v):
    """Candidates for one (Br, Bc) in reference order: register then shared, per knob setting."""
    out = []
    for slab_qk, st_qk in _qk_slabs(dim_qk):
        if slab_qk % 32:
            continue
        for slab_v, st_v in _v_slabs(bc):
            if slab_v % 32:
                continue
            for nthreads in _THREADS:
                if not _thread_rule_ok(br, bc, slab_qk, slab_v, nthreads):
                    continue
                for unroll in (True, False):
                    for fuse in ("register", "shared"):
                        if op == "attn":
                            cfg = AttnConfig(br, bc, dim_qk, dim_v, slab_qk, slab_v, st_qk, st_v, nthreads, unroll)
                        else:
                            cfg = RetConfig(br, bc, dim_qk, dim_v, slab_qk, slab_v, st_qk, 1, st_v, nthreads, unroll)
                        out.append(cfg.set_fuse_type(fuse))
    return out


def _stage_bytes(cfg):
    qk = cfg.num_stages_qk * (cfg.Br + cfg.Bc) * cfg.BlockKSmem * 2
    v = cfg.num_stages_v * cfg.BlockKSmem2 * cfg.D * 2
    mask = cfg.num_stages_mask * cfg.Br * cfg.Bc * 2 if cfg.operation == "ret" else 0
    return qk + v + mask


def _reg_limit(arch, nthreads):
    return min(arch.register_per_thread, arch.reg_cap / nthreads)


def forward_valid(cfg, arch):
    out_bytes = cfg.Br * cfg.D * 2
    if cfg.fuse_type == "register":
        mma_m = arch.cutlass_mma[0]
        if cfg.Br % (mma_m * cfg.Nthreads / arch.warp_size):
            return False
        if max(_stage_bytes(cfg), out_bytes) > arch.smem_cap:
            return False
        acc_regs = (cfg.Br * cfg.D * 4 + cfg.Br * cfg.Bc * 4) / (cfg.Nthreads * 4)
        return acc_regs <= _reg_limit(arch, cfg.Nthreads)
    # shared fuse: S (fp32) + P (fp16) + per-row statistics live in shared memory
    stats = (3 if cfg.operation == "attn" else 2) * cfg.Br * 4
    accs = cfg.Br * cfg.Bc * 2 + cfg.Br * cfg.Bc * 4 + stats
    if max(_stage_bytes(cfg) + accs, out_bytes) > arch.smem_cap:
        return False
    return (cfg.Br * cfg.D * 4) / (cfg.Nthreads * 4) <= _reg_limit(arch, cfg.Nthreads)


def backward_candidates(br, bc, dim_qk, dim_v):
    out = []
    if br < 64 or bc < 64:
        return out
    for nthreads in _THREADS:
        n_warps = nthreads // 32
        splits = [balanced_wave_split(n_warps, r, c) for r, c in ((br, bc), (bc, dim_v), (bc, dim_qk), (br, dim_qk))]
        if any(s is None for s in splits) or dim_qk % 32:
            continue
        n_s, n_dv, n_dk, n_dq = (s[1] for s in splits)
        for unroll in (True, False):
            out.append(RetBwdConfig(br, bc, dim_qk, dim_v, n_s, n_dv, n_dk, n_dq, nthreads, unroll,
                                    BlockKSmem=dim_qk, num_stages_qk=1))
    return out


def backward_valid(cfg, arch):
    qk = cfg.num_stages_qk * (cfg.Br + cfg.Bc) * cfg.BlockKSmem * 2
    mask = cfg.num_stages_mask * cfg.Br * cfg.Bc * 2
    s_do = cfg.Br * cfg.Bc * 2 + cfg.Br * cfg.D * 2
    v = cfg.Bc * cfg.D * 2
    return qk + mask + s_do + v <= arch.smem_cap
