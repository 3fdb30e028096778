"""Host-side bounds check of the LDS-patch convolution kernels' global loads (CPU only, no GPU).

The staging code of ferrox_amd/csrc/wgrad_patch.hpp and conv_patch.hpp computes every global address as a
wave-uniform base plus a per-thread offset; lanes and 16-row passes that fall outside the tile's data are redirected to
an address that is known to be mapped.  This file restates that address arithmetic (and the planners that pick the
tile) and walks it for every thread of every block for the shapes of the GPU tests: each 16-byte load must lie inside
its tensor.  It guards the fix of an over-read: passes of grad_out rows that start past the last output channel used to
be read up to 53 KB past the end of the tensor in the last image.
"""
import pytest

LPR, NT, RPP = 16, 256, 16
def _odd_pitch_w(n): return (n + 30) // 32 * 32 + 1
def wgrad_plan(num_cus, B, Cin, H, W, Cout, sh, sw, ph, pw, oh, ow):
    if Cin % 32 and (Cout > 32 or (Cin + 31) // 32 * 32 > 2 * Cin): return None
    if ow % 2 or W % 4 or W > 64 or sh > 8 or sw > 8: return None
    cand = []
    if Cout <= 32:
        if Cin % 64 == 0 and ow % 4 == 0: cand.append((1, 2, 2))
        if ow % 8 == 0: cand.append((1, 1, 4))
    elif Cout <= 64:
        if Cin % 64 == 0: cand.append((2, 2, 1))
        if ow % 4 == 0: cand.append((2, 1, 2))
    else:
        cand.append((4, 1, 1))
    best = 0
    for WMO, WC, WK in cand:
        BM, CT = 32 * WMO, 32 * WC
        max_pr = 3 if WC == 2 else 4
        for R in range(1, oh + 1):
            if oh % R or R * ow > 64 or (R - 1) * sh + 3 > max_pr: continue
            if (R * ow) % 4 == 0: best = R
        if best * ow < 24: best = 0
        if best:
            PR = (best - 1) * sh + 3
            smem = (BM * _odd_pitch_w(best * ow) + CT * _odd_pitch_w(PR * (W + 2 * pw)) + 64) * 4
            if WK > 1: smem = max(smem, 4 * 16 * 64 * 4)
            if smem > 72 * 1024: best = 0
        if best: break
    if not best:
        # maps of at most 64 pixels with rows of at most 16 floats: one whole image per stage, (channel, row) pair staging
        L, XRn = oh * ow, (oh - 1) * sh + 3
        if Cout > 64: WMO, WK = 4, 1
        elif Cout > 32 and ow % 4 == 0: WMO, WK = 2, 2
        elif Cout <= 32 and ow % 8 == 0: WMO, WK = 1, 4
        else: return None
        if W > 16 or L > 64 or L < 24 or L % 4 or XRn > 10: return None
        return dict(R=oh, PR=XRn, BM=32 * WMO, CT=32, Kst=L, stages=B, spi=1, narrow=True)
    PR = (best - 1) * sh + 3
    return dict(R=best, PR=PR, BM=BM, CT=CT, Kst=best * ow, stages=B * (oh // best), spi=oh // best, narrow=False)
def wgrad_loads_in_bounds(B, Cin, H, W, Cout, st, pd):
    sh, sw = st; ph, pw = pd
    oh, ow = (H + 2 * ph - 3) // sh + 1, (W + 2 * pw - 3) // sw + 1
    pl = wgrad_plan(256, B, Cin, H, W, Cout, sh, sw, ph, pw, oh, ow)
    if pl is None: return "generic"
    L = oh * ow
    gsize, xsize = B * Cout * L, B * Cin * H * W
    k4, w4 = pl["Kst"] // 4, W // 4
    NG, NXC = pl["BM"] // RPP, pl["CT"] // RPP
    for s in range(pl["stages"]):
        b = s // pl["spi"]; oy0 = (s - b * pl["spi"]) * pl["R"]; iy0 = oy0 * sh - ph
        for oc0 in range(0, Cout, pl["BM"]):
            full_m = oc0 + pl["BM"] <= Cout
            gsrc = (b * Cout + oc0) * L + oy0 * ow
            for tid in range(NT):
                pq, prow = tid % LPR, tid // LPR
                g_off = (prow * L + 4 * pq) if pq < k4 else 0
                for u in range(NG):
                    ok = full_m or oc0 + prow + u * RPP < Cout
                    pass_in = full_m or oc0 + u * RPP < Cout
                    base = gsrc + u * RPP * L if pass_in else gsrc
                    a = base + (g_off if ok else 0)
                    assert 0 <= a and a + 4 <= gsize, ("g", (B, Cin, H, W, Cout, st, pd), s, oc0, tid, u, a, gsize)
                    if ok and pq < k4:  # the four floats are pixels of this stage in the lane's own channel row
                        row0 = (b * Cout + oc0 + prow + u * RPP) * L + oy0 * ow
                        assert row0 <= a and a + 4 <= row0 + pl["Kst"]
        for c0 in (range(0, Cin, pl["CT"]) if pl["narrow"] else ()):
            xsrc = (b * Cin + c0) * H * W
            full_c = c0 + pl["CT"] <= Cin
            PW = W + 2 * pw; PLANE = _odd_pitch_w(pl["PR"] * PW)
            for tid in range(NT):
                npq, npp = tid & 3, tid >> 2
                lane_in = npq < ((W + 3) >> 2); col = min(4 * npq, W - 4)
                for u in range(5):
                    pair = u * 64 + npp; c, r = divmod(pair, pl["PR"]); iy = iy0 + r
                    ok = lane_in and pair < pl["CT"] * pl["PR"] and 0 <= iy < H and (full_c or c0 + c < Cin)
                    a = xsrc + (((c * H + iy) * W + col) if ok else 0)
                    assert 0 <= a and a + 4 <= xsize, ("x narrow", a, xsize)
                    if ok:
                        row0 = ((b * Cin + c0 + c) * H + iy) * W
                        assert row0 <= a and a + 4 <= row0 + W
                    if lane_in and pair < pl["CT"] * pl["PR"] and (full_c or c0 + c < Cin):
                        d = c * PLANE + r * PW + pw + col
                        assert 0 <= d and d + 4 <= pl["CT"] * PLANE, ("Xs narrow", d)
        for c0 in (() if pl["narrow"] else range(0, Cin, pl["CT"])):
            xsrc = (b * Cin + c0) * H * W
            full_c = c0 + pl["CT"] <= Cin
            for tid in range(NT):
                pq, prow = tid % LPR, tid // LPR
                xcol = 4 * pq
                x_off = (prow * H * W + xcol) if pq < w4 else 0
                x_off0 = xcol if pq < w4 else 0
                for r in range(pl["PR"]):
                    iy = iy0 + r
                    if not (0 <= iy < H): continue
                    for cu in range(NXC):
                        pass_in = full_c or c0 + cu * RPP < Cin
                        ok = full_c or c0 + prow + cu * RPP < Cin
                        a = xsrc + ((cu * RPP if pass_in else 0) * H + iy) * W + (x_off if ok else x_off0)
                        assert 0 <= a and a + 4 <= xsize, ("x", (B, Cin, H, W, Cout, st, pd), a, xsize)
                        if ok and pq < w4:  # the plane read is the one the lane parks
                            assert a == ((b * Cin + c0 + cu * RPP + prow) * H + iy) * W + xcol and xcol + 4 <= W
    return "patch"

CC, KK, WPITCH = 8, 9, 73
NXP_SHORT, NXP_TALL = 4, 10
PPLANE = 1149   # fixed plane pitch of the persistent variant
def _ceil_div(a, b): return (a + b - 1) // b
def _odd_pitch_c(n): return (n + 30) // 32 * 32 + 1
def fwd_plan(num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw):
    if C % CC or W < 4 or W > 4 * LPR or sh > 8 or sw > 8: return None
    L, slots = OH * OW, 2 * num_cus
    RPI = (OH - 1) * sh + 3
    if L <= 64 and B >= 2:  # small maps: whole images stacked in one tile
        nimg = min(128 // L, 2 * NXP_TALL // RPI, B)
        wm = 4 if M > 64 else 2
        bm = 32 * wm; mtiles = _ceil_div(M, bm)
        if nimg >= 2 and nimg * L >= 64 and mtiles * bm <= M * 2:
            PR = nimg * RPI; PW = W + 2 * pw; PLANE = _odd_pitch_c(PR * PW)
            if (bm * WPITCH + CC * PLANE + 16) * 4 > 72 * 1024: return None
            return [dict(WM=wm, TN=4 if wm == 4 else 2, PR=PR, tpi=1, mtiles=mtiles, nchunks=C // CC, BM=bm, NPIX=128, NXP=NXP_TALL,
                         nimg=nimg, RPI=RPI, PW=PW, PLANE=PLANE, cost=0)]
    plans = []
    for wm, tn in [(4, 8), (4, 7), (4, 6), (4, 5), (4, 4), (2, 4), (2, 3), (2, 2), (1, 4), (1, 3), (1, 2)]:
        bm, np_ = 32 * wm, 32 * tn * (4 // wm)
        tiles, mtiles = _ceil_div(L, np_), _ceil_div(M, bm)
        rows = min(OH, np_ // OW if np_ % OW == 0 else (np_ - 1) // OW + 2); PR = (rows - 1) * sh + 3
        tall_ok = wm <= 2 or tn <= 6
        if PR > 2 * NXP_TALL or (PR > 2 * NXP_SHORT and not tall_ok) or mtiles * bm > M * 2 or tiles * np_ > L * 2: continue
        PW = W + 2 * pw; PLANE = _odd_pitch_c(PR * PW)
        if (bm * WPITCH + CC * PLANE + 16) * 4 > 72 * 1024: continue
        cost = _ceil_div(B * tiles * mtiles, slots) * np_ * bm
        plans.append(dict(WM=wm, TN=tn, PR=PR, tpi=tiles, mtiles=mtiles, nchunks=C // CC, BM=bm, NPIX=np_, cost=cost,
                          NXP=NXP_TALL if PR > 2 * NXP_SHORT else NXP_SHORT))
    return plans or None
def fwd_multi_loads_in_bounds(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw):
    L, xsize, ysize = OH * OW, B * C * H * W, B * M * OH * OW
    nimg, RPI, PR, PW = pl["nimg"], pl["RPI"], pl["PR"], pl["PW"]
    for bx in range(_ceil_div(B, nimg)):
        b0 = bx * nimg
        for ch in range(pl["nchunks"]):
            for tid in range(NT):
                pq, xc, rp = tid & 15, (tid >> 4) & 7, tid >> 7
                lane_in = pq < ((W + 3) >> 2)
                x_off = (xc * H * W + min(4 * pq, W - 4)) if lane_in else 0
                for u in range(pl["NXP"]):
                    r = 2 * u + rp; img = r // RPI; iy = r - img * RPI - ph
                    if r < PR and 0 <= iy < H and b0 + img < B:
                        a = (b0 * C + ch * CC) * H * W + (img * C * H + iy) * W + x_off
                        assert 0 <= a and a + 4 <= xsize, ("x", a, xsize)
                        if lane_in:
                            row0 = (((b0 + img) * C + ch * CC + xc) * H + iy) * W
                            assert row0 <= a and a + 4 <= row0 + W
        for pi in range(pl["NPIX"]):  # LDS offsets of the pixels and the addresses they are stored to
            img, rem = divmod(pi, L); py, px = divmod(rem, OW)
            if img < nimg and b0 + img < B:
                assert (img * RPI + py * sh + 2) * PW + px * sw + 2 < PR * PW <= pl["PLANE"]
                assert ((b0 + img) * M + (M - 1)) * L + rem < ysize
    return "patch multi %dx%d ok" % (pl["WM"], pl["TN"])
def fwd_loads_in_bounds(B, C, H, W, M, sh, sw, ph, pw):
    OH, OW = (H + 2 * ph - 3) // sh + 1, (W + 2 * pw - 3) // sw + 1
    plans = fwd_plan(256, B, C, H, W, M, OH, OW, sh, sw, ph, pw)
    if plans is None: return "generic"
    # every tile shape that fits is walked: the library times the candidates once per layer shape and keeps the fastest
    out = [fwd_shape_loads_in_bounds(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw) for pl in plans]
    if not plans[0].get("nimg"):
        out += [persist_walk(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw) for pl in persist_plans(B, C, H, W, M, OH, OW, sh, sw, ph, pw)]
    return " ".join(out)
def fwd_shape_loads_in_bounds(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw):
    if pl.get("nimg"): return fwd_multi_loads_in_bounds(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw)
    WIMG = pl["BM"] * WPITCH
    NW = (WIMG // 4 + NT - 1) // NT
    wbuf = pl["mtiles"] * pl["nchunks"] * WIMG          # floats written by wimg_kernel
    xsize = B * C * H * W
    for b in (0, B - 1):
        for tile in range(pl["tpi"]):
            pix0 = tile * pl["NPIX"]; py0 = pix0 // OW; iy_base = py0 * sh - ph
            for my in range(pl["mtiles"]):
                for ch in range(pl["nchunks"]):
                    wsrc = my * pl["nchunks"] * WIMG + ch * WIMG
                    xsrc = b * C * H * W + ch * CC * H * W
                    for tid in range(NT):
                        for u in range(NW):
                            idx = tid + u * NT
                            idx = idx if ((u + 1) * NT <= WIMG // 4 or idx < WIMG // 4) else 0
                            a = wsrc + idx * 4
                            assert 0 <= a and a + 4 <= wbuf, ("w", a, wbuf)
                        pq, xc, rp = tid & 15, (tid >> 4) & 7, tid >> 7
                        x_off = (xc * H * W + min(4 * pq, W - 4)) if pq < ((W + 3) >> 2) else 0
                        for u in range(pl["NXP"]):
                            r = 2 * u + rp; iy = iy_base + r
                            if r < pl["PR"] and 0 <= iy < H:
                                a = xsrc + iy * W + x_off
                                assert 0 <= a and a + 4 <= xsize, ("x", (B, C, H, W, M), a, xsize)
                                if pq < ((W + 3) >> 2):  # the four floats lie inside row iy of channel xc
                                    row0 = ((b * C + ch * CC + xc) * H + iy) * W
                                    assert row0 <= a and a + 4 <= row0 + W
    return "patch %dx%d ok" % (pl["WM"], pl["TN"])


NXP_PERSIST = 5
def persist_plans(B, C, H, W, M, OH, OW, sh, sw, ph, pw):
    """The tile shapes of conv_patch_persist_kernel that fit a layer (persist_plan)."""
    L, plans = OH * OW, []
    for wm, tn in [(4, 5), (4, 4), (2, 5), (2, 4), (2, 3)]:
        bm, np_ = 32 * wm, 32 * tn * (4 // wm)
        tiles, mtiles = _ceil_div(L, np_), _ceil_div(M, bm)
        rows = min(OH, np_ // OW if np_ % OW == 0 else (np_ - 1) // OW + 2); PR = (rows - 1) * sh + 3
        if PR > 2 * NXP_PERSIST or mtiles * bm > M * 2 or tiles * np_ > L * 2: continue
        pw2 = W + 2 * pw
        if sw == 1:
            padded = pw2
            while (sh * padded - OW) % 32: padded += 1
            if PR * padded <= PPLANE: pw2 = padded
        if PR * pw2 > PPLANE: continue
        plans.append(dict(WM=wm, TN=tn, PR=PR, tpi=tiles, mtiles=mtiles, nchunks=C // CC, BM=bm, NPIX=np_, PW=pw2))
    return plans
def persist_walk(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw, num_cus=256):
    """conv_patch_persist_kernel: the blocks' tile sequences cover every tile exactly once; weight-image, input and output
    addresses and the LDS offsets of every tile stay inside their buffers."""
    PW, PLANE, bufsz = pl["PW"], PPLANE, CC * PPLANE + 16
    assert PLANE % 4 == 1 and PLANE >= pl["PR"] * PW and PW >= W + 2 * pw and pl["PR"] <= 2 * NXP_PERSIST
    L, WM, TN, NPIX = OH * OW, pl["WM"], pl["TN"], pl["NPIX"]
    bt = B * pl["tpi"]; ntiles = bt * pl["mtiles"]
    nblk = min(ntiles, 2 * num_cus); chunk = 0      # two blocks per CU
    if ntiles % 8 == 0 and nblk >= 8:
        nblk -= nblk % 8; chunk = ntiles // 8
    seen = [0] * ntiles
    for bid in range(nblk):
        if chunk: x = bid & 7; q, step, end = x * chunk + (bid >> 3), nblk >> 3, (x + 1) * chunk
        else: q, step, end = bid, nblk, ntiles
        while q < end:
            seen[q] += 1; q += step
    assert all(v == 1 for v in seen), "tiles visited %s" % sorted(set(seen))
    wbuf2 = pl["mtiles"] * WM * pl["nchunks"] * KK * 64 * 4            # floats written by wimg2_kernel
    assert wbuf2 * 4 <= _ceil_div(M, 128) * 128 * WPITCH * pl["nchunks"] * 4   # the workspace the entry point asks for
    xsize, ysize = B * C * H * W, B * M * L
    tiles = sorted({0, 1, pl["tpi"] - 1, pl["tpi"], bt - 1, ntiles - 1, ntiles // 2} & set(range(ntiles)))
    for q in tiles:
        mt, rem = divmod(q, bt); b, t = divmod(rem, pl["tpi"])
        pix0 = t * NPIX; py0 = pix0 // OW; iy_base = py0 * sh - ph; m0 = mt * pl["BM"]
        for wm in range(WM):
            for ch in (0, pl["nchunks"] - 1):
                a = ((mt * WM + wm) * pl["nchunks"] + ch) * KK * 64 * 4 + (8 * 64 + 63) * 4
                assert a + 4 <= wbuf2, ("A", a, wbuf2)
        for ch in (0, pl["nchunks"] - 1):
            for tid in range(NT):
                pq, xc, rp = tid & 15, (tid >> 4) & 7, tid >> 7
                lane_in = pq < ((W + 3) >> 2); xcol = min(4 * pq, W - 4)
                for u in range(NXP_PERSIST):
                    r = 2 * u + rp; iy = iy_base + r
                    if r < pl["PR"] and 0 <= iy < H:
                        a = ((b * C + ch * CC) * H + iy) * W + ((xc * H * W + xcol) if lane_in else 0)
                        assert 0 <= a and a + 4 <= xsize, ("x", a, xsize)
                    if r < pl["PR"] and lane_in:
                        d = xc * PLANE + pw + xcol + r * PW
                        assert 0 <= d and d + 4 <= CC * PLANE, ("park", d)
        for pi in range(pix0, pix0 + NPIX):
            if pi >= L: continue
            py, px = divmod(pi, OW)
            off = (py - py0) * sh * PW + px * sw + 7 * PLANE + 2 * PW + 2   # last channel pair, last tap
            assert 0 <= (py - py0) * sh + 2 < pl["PR"] and px * sw + 2 < PW and off < CC * PLANE, ("B read", off)
            assert (bufsz + 6 * PLANE + 2) * 4 < 65536   # buffer + channel pair + filter column ride in a read's 16-bit offset field
            assert 2 * bufsz * 4 <= 72 * 1024            # two buffers
            assert (b * M + min(M, m0 + pl["BM"]) - 1) * L + pi < ysize
    return "persist %dx%d ok" % (WM, TN)


# ---- conv_smallc.hpp: image layers (few input channels), forward and weight gradient ------------------------------------
SC_NPIX, SC_GP = 256, 257
def smallc_plan(wgrad, B, C, H, W, Cout, sh, sw, ph, pw, OH, OW, num_cus=256):
    L = OH * OW
    if W < 4 or sh > 8 or sw > 8 or ph > 8 or pw > 8: return None
    if (C * 9 > 32 or L % 4) if wgrad else C > 4: return None
    rows = min(OH, SC_NPIX // OW if SC_NPIX % OW == 0 else (SC_NPIX - 1) // OW + 2)
    PR, PW = (rows - 1) * sh + 3, W + 2 * pw
    if OW > 64 or PR * OW > 2 * SC_NPIX * sh: return None
    pl = dict(PR=PR, PW=PW, PLANE=PR * PW, tpi=_ceil_div(L, SC_NPIX))
    if (C * pl["PLANE"] + (32 * SC_GP if wgrad else 0)) * 4 > 60 * 1024: return None
    if not wgrad and C * PR * ((W + 3) // 4) > 4 * 256: return None   # the patch items a thread of the forward kernel keeps in flight
    if wgrad:
        stages, mblocks = B * pl["tpi"], _ceil_div(Cout, 32)
        splits = max(1, min(stages, 4 * num_cus // mblocks))
        pl["sps"] = _ceil_div(stages, splits); pl["splits"] = _ceil_div(stages, pl["sps"]); pl["stages"] = stages
    return pl
def smallc_tap(C, PLANE, PW, k):
    if k >= C * 9: return 0
    c, t = divmod(k, 9); ky, kx = divmod(t, 3)
    return c * PLANE + ky * PW + kx
def smallc_stage_in_bounds(pl, b, C, H, W, pw, iy0, xsize):
    W4 = (W + 3) // 4
    for i in range(C * pl["PR"] * W4):
        rc, q = divmod(i, W4); c, r = divmod(rc, pl["PR"])
        q = min(4 * q, W - 4)
        iy = iy0 + r; ok = 0 <= iy < H
        a = ((b * C + c) * H + (iy if ok else 0)) * W + q
        assert 0 <= a and a + 4 <= xsize, ("x", a, xsize)
        d = c * pl["PLANE"] + r * pl["PW"] + pw + q
        assert 0 <= d and d + 4 <= C * pl["PLANE"], ("patch write", d)
def smallc_loads_in_bounds(wgrad, B, C, H, W, Cout, st, pd):
    sh, sw = st; ph, pw = pd
    OH, OW = (H + 2 * ph - 3) // sh + 1, (W + 2 * pw - 3) // sw + 1
    pl = smallc_plan(wgrad, B, C, H, W, Cout, sh, sw, ph, pw, OH, OW)
    if pl is None: return "generic"
    L, K = OH * OW, C * 9
    xsize, ysize, wsize = B * C * H * W, B * Cout * L, Cout * K
    KS = {1: 5, 2: 9, 3: 14, 4: 18}[C]
    plane_all = C * pl["PLANE"]
    for b in range(B):
        for tile in range(pl["tpi"]):
            pix0 = tile * SC_NPIX; py0 = pix0 // OW; iy0 = py0 * sh - ph
            smallc_stage_in_bounds(pl, b, C, H, W, pw, iy0, xsize)
            for m0 in range(0, Cout, 32):
                if not wgrad:
                    for l32 in range(32):
                        m_ok = m0 + l32 < Cout
                        for k in range(2 * KS):
                            a = (m0 + l32 if m_ok else 0) * K + (k if k < K else 0)
                            assert 0 <= a < wsize, ("w", a)
                    for pb in range(8):
                        pbase = pix0 + pb * 32
                        if pbase >= L: break
                        for l32 in range(32):
                            pp = pbase + l32; pc = min(pp, L - 1); oy, ox = divmod(pc, OW)
                            assert (oy - py0) * sh + 2 < pl["PR"], "patch rows"
                            base = (oy - py0) * sh * pl["PW"] + ox * sw
                            for k in range(2 * KS):
                                idx = base + smallc_tap(C, pl["PLANE"], pl["PW"], k)
                                assert 0 <= idx < plane_all, ("patch read", idx)
                            if pp < L:
                                for ch in range(m0, min(m0 + 32, Cout)):
                                    a = (b * Cout + ch) * L + pp
                                    assert 0 <= a < ysize
                else:
                    for tid in range(256):
                        gq, gr = tid & 63, tid >> 6
                        col_ok = pix0 + 4 * gq < L
                        for u in range(8):
                            row = gr + 4 * u; ok = col_ok and m0 + row < Cout
                            a = (b * Cout + (m0 + row if ok else 0)) * L + (pix0 + 4 * gq if ok else 0)
                            assert 0 <= a and a + 4 <= ysize, ("g", a, ysize)
                            assert row * SC_GP + 4 * gq + 4 <= 32 * SC_GP
                    for wave in range(4):
                        for half in range(2):
                            for stp in range(32):
                                pl_ = wave * 64 + half + 2 * stp
                                assert pl_ < SC_NPIX
                                pc = min(pix0 + pl_, L - 1); oy, ox = divmod(pc, OW)
                                assert (oy - py0) * sh + 2 < pl["PR"], "patch rows"
                                base = (oy - py0) * sh * pl["PW"] + ox * sw
                                for n in range(32):
                                    idx = base + smallc_tap(C, pl["PLANE"], pl["PW"], n)
                                    assert 0 <= idx < plane_all, ("patch read", idx)
    if wgrad:
        assert pl["splits"] * pl["sps"] >= pl["stages"] and (pl["splits"] - 1) * pl["sps"] < pl["stages"]
    return "smallc"


SMALLC_SHAPES = [  # B, C, H, W, Cout, (sh, sw), (ph, pw)
    (2, 3, 32, 32, 32, (1, 1), (1, 1)), (2, 1, 28, 28, 8, (1, 1), (1, 1)), (3, 3, 9, 12, 40, (1, 1), (0, 0)),
    (2, 2, 17, 20, 33, (2, 2), (1, 1)), (2, 3, 7, 8, 5, (3, 1), (1, 1)), (1, 3, 40, 36, 64, (1, 1), (1, 1)),
    (1, 3, 66, 64, 16, (2, 2), (1, 1)), (2, 1, 5, 4, 70, (1, 1), (2, 2)), (1, 3, 19, 60, 8, (1, 1), (1, 1)),
    (2, 3, 14, 14, 32, (1, 1), (1, 1)), (2, 1, 9, 7, 16, (1, 1), (1, 1)), (2, 3, 12, 30, 8, (1, 1), (1, 1)),
]


@pytest.mark.parametrize("case", SMALLC_SHAPES, ids=str)
def test_image_layer_kernels_stay_inside_their_tensors_and_the_patch(case):
    B, C, H, W, Cout, (sh, sw), (ph, pw) = case
    L = ((H + 2 * ph - 3) // sh + 1) * ((W + 2 * pw - 3) // sw + 1)
    assert smallc_loads_in_bounds(False, *case) == "smallc"
    assert smallc_loads_in_bounds(True, *case) == ("smallc" if L % 4 == 0 else "generic")  # whole float4 groups of grad_out


def test_image_layer_forward_takes_four_channels_and_the_weight_gradient_does_not():
    case = (1, 4, 10, 64, 16, (1, 2), (2, 0))
    assert smallc_loads_in_bounds(False, *case) == "smallc"
    assert smallc_loads_in_bounds(True, *case) == "generic"


WGRAD_SHAPES = [  # B, Cin, H, W, Cout, (sh, sw), (ph, pw): every wave layout, ragged output-channel counts
    (2, 32, 10, 56, 100, (1, 1), (1, 1)), (3, 64, 28, 28, 96, (1, 1), (1, 1)), (2, 32, 16, 16, 128, (1, 1), (1, 1)),
    (2, 32, 9, 64, 128, (1, 1), (0, 1)), (2, 64, 12, 56, 64, (1, 1), (1, 1)), (3, 64, 10, 32, 64, (1, 1), (1, 1)),
    (2, 32, 12, 32, 64, (1, 1), (1, 1)), (5, 32, 6, 64, 33, (1, 1), (1, 1)), (1, 32, 6, 24, 40, (1, 1), (1, 1)),
    (2, 64, 6, 28, 49, (1, 1), (1, 1)), (1, 32, 4, 32, 97, (1, 1), (1, 1)), (3, 32, 8, 12, 72, (1, 1), (1, 1)),
    (2, 32, 8, 16, 150, (1, 1), (1, 1)), (1, 64, 5, 56, 36, (1, 1), (1, 1)), (2, 32, 8, 56, 65, (2, 1), (1, 1)),
    # at most 32 output channels: 1 x 2 x 2 and 1 x 1 x 4, ragged counts
    (2, 64, 8, 32, 32, (1, 1), (1, 1)), (3, 32, 8, 32, 32, (1, 1), (1, 1)), (2, 64, 6, 28, 20, (1, 1), (1, 1)), (2, 32, 10, 24, 7, (1, 1), (1, 1)),
    (2, 96, 12, 16, 17, (1, 1), (1, 1)), (2, 128, 16, 16, 32, (1, 1), (1, 1)), (2, 128, 16, 16, 64, (1, 1), (1, 1)),
    # input channels that do not fill the last block of 32
    (2, 16, 8, 32, 32, (1, 1), (1, 1)), (3, 48, 8, 32, 30, (1, 1), (1, 1)), (2, 24, 12, 24, 20, (1, 1), (1, 1)), (2, 40, 6, 16, 13, (1, 1), (1, 1)),
    (1, 33, 8, 24, 16, (1, 1), (1, 1)), (2, 17, 6, 32, 32, (1, 1), (1, 1)),
    # 64 x 64 channels at 64-wide rows: the 64-plane layout exceeds the LDS budget, the 32-plane one is taken
    (2, 64, 8, 64, 64, (1, 1), (1, 1)), (2, 64, 8, 64, 32, (1, 1), (1, 1)),
    # narrow maps: one whole image per stage
    (3, 64, 8, 8, 128, (1, 1), (1, 1)), (2, 32, 8, 8, 64, (1, 1), (1, 1)), (2, 96, 8, 8, 20, (1, 1), (1, 1)), (2, 32, 6, 8, 100, (1, 1), (1, 1)),
    (3, 64, 4, 16, 72, (1, 1), (1, 1)), (2, 48, 8, 8, 24, (1, 1), (1, 1)),
]
FWD_SHAPES = [  # B, C, H, W, M, (sh, sw), (ph, pw): one per tile shape on a 256-CU device, ragged M, strides, paddings
    (2, 64, 28, 28, 64, (1, 1), (1, 1)), (2, 8, 6, 12, 60, (1, 1), (1, 1)), (3, 16, 8, 36, 120, (1, 1), (0, 0)),
    (2, 24, 6, 8, 104, (1, 1), (2, 2)), (1, 8, 64, 64, 52, (1, 1), (1, 1)), (2, 16, 15, 18, 60, (2, 2), (1, 1)),
    (2, 8, 9, 64, 128, (2, 1), (1, 1)), (128, 8, 8, 40, 120, (1, 1), (1, 1)), (32, 8, 56, 56, 64, (1, 1), (1, 1)),
    (16, 8, 56, 56, 120, (1, 1), (1, 1)), (128, 8, 8, 40, 250, (1, 1), (1, 1)), (96, 8, 12, 48, 384, (1, 1), (1, 1)),
    (32, 8, 56, 56, 120, (1, 1), (1, 1)), (128, 8, 16, 64, 120, (1, 1), (1, 1)),
    # strided layers: more than 8 patch rows under a tile
    (8, 32, 32, 32, 64, (2, 2), (1, 1)), (4, 64, 56, 56, 128, (2, 2), (1, 1)), (2, 16, 30, 40, 60, (2, 1), (1, 1)),
    (2, 8, 16, 34, 128, (3, 3), (1, 1)), (64, 64, 56, 56, 128, (2, 2), (1, 1)),
    # 32 output channels: one block of channels, four waves along the pixels
    (256, 64, 32, 32, 32, (1, 1), (1, 1)), (3, 16, 9, 20, 30, (1, 1), (1, 1)), (64, 8, 16, 32, 32, (2, 1), (1, 1)), (2, 8, 18, 10, 27, (1, 1), (0, 0)),
    # up to half of a tile's channel rows are padding
    (2, 16, 8, 32, 16, (1, 1), (1, 1)), (2, 8, 12, 28, 40, (1, 1), (1, 1)), (128, 8, 56, 56, 72, (1, 1), (1, 1)), (3, 24, 12, 12, 17, (1, 1), (1, 1)),
    # row lengths that are not multiples of four floats
    (3, 8, 14, 14, 64, (1, 1), (1, 1)), (2, 16, 10, 7, 32, (1, 1), (1, 1)), (2, 8, 9, 30, 128, (1, 1), (0, 0)), (2, 8, 15, 18, 40, (2, 2), (1, 1)),
    (2, 8, 6, 63, 64, (1, 1), (1, 1)),
    # maps of at most 64 pixels: whole images stacked in one tile (odd batch: the last tile holds one image)
    (5, 16, 8, 8, 128, (1, 1), (1, 1)), (3, 8, 7, 7, 64, (1, 1), (1, 1)), (7, 8, 6, 6, 40, (1, 1), (1, 1)), (4, 8, 6, 10, 200, (1, 1), (0, 1)),
    (5, 8, 16, 16, 64, (2, 2), (1, 1)), (2, 8, 8, 8, 33, (1, 1), (2, 2)),
]


@pytest.mark.parametrize("case", WGRAD_SHAPES, ids=str)
def test_weight_gradient_patch_kernel_loads_stay_inside_the_tensors(case):
    B = min(case[0], 3)  # the first and the last images are the ones at the tensor ends
    assert wgrad_loads_in_bounds(B, *case[1:]) == "patch", "the shape must exercise the patch kernel"


@pytest.mark.parametrize("case", FWD_SHAPES, ids=str)
def test_forward_patch_kernel_loads_stay_inside_the_tensors(case):
    B, C, H, W, M, st, pd = case
    assert fwd_loads_in_bounds(B, C, H, W, M, st[0], st[1], pd[0], pd[1]).startswith("patch")
    if st == (1, 1):  # the data gradient runs the same kernel over grad_out with padding 2 - p and channels swapped
        OH, OW = H + 2 * pd[0] - 2, W + 2 * pd[1] - 2
        fwd_loads_in_bounds(B, M, OH, OW, C, 1, 1, 2 - pd[0], 2 - pd[1])


# ---- conv_patch_f64.hpp: the f64 twin of the persistent forward / data-gradient kernel ---------------------------------------
D_PPLANE, D_NXP, D_LPR = 573, 8, 32
def f64_plans(B, C, H, W, M, OH, OW, kh, kw, sh, sw, ph, pw):
    """cpd::make_plan's candidates (tile widths 8, 7, 5), or [] when the layer stays on the implicit GEMM."""
    L = OH * OW
    if kh != 3 or kw != 3 or C % CC or W < 2 or W % 2 or W > 2 * D_LPR or sh > 8 or sw > 8 or L < 64 or M < 32: return []
    plans = []
    for tn in (8, 7, 5):
        np_ = 16 * tn
        tiles, mtiles = _ceil_div(L, np_), _ceil_div(M, 64)
        rows = min(OH, np_ // OW if np_ % OW == 0 else (np_ - 1) // OW + 2); PR = (rows - 1) * sh + 3
        if PR > D_NXP or mtiles * 64 > M * 2 or tiles * np_ > L * 2: continue
        pw2 = W + 2 * pw
        if sw == 1:
            padded = pw2
            while (sh * padded - OW) % 16: padded += 1
            if PR * padded <= D_PPLANE: pw2 = padded
        if PR * pw2 > D_PPLANE: continue
        plans.append(dict(TN=tn, PR=PR, PW=pw2, tpi=tiles, mtiles=mtiles, nchunks=C // CC, NPIX=np_))
    return plans
def f64_walk(pl, B, C, H, W, M, OH, OW, sh, sw, ph, pw, num_cus=256):
    """Every tile is visited exactly once; weight-image, input and output addresses and the LDS offsets stay inside their buffers;
    every 16-byte load is 16-byte aligned."""
    PW, PLANE, bufsz, L, NPIX = pl["PW"], D_PPLANE, CC * D_PPLANE + 16, OH * OW, pl["NPIX"]
    assert PLANE >= pl["PR"] * PW and PW >= W + 2 * pw and pl["PR"] <= D_NXP
    assert 2 * bufsz * 8 <= 72 * 1024 and (bufsz + 4 * PLANE + 2) * 8 < 65536
    bt = B * pl["tpi"]; ntiles = bt * pl["mtiles"]
    nblk = min(ntiles, 2 * num_cus); chunk = 0
    if ntiles % 8 == 0 and nblk >= 8:
        nblk -= nblk % 8; chunk = ntiles // 8
    seen = [0] * ntiles
    for bid in range(nblk):
        if chunk: x = bid & 7; q, step, end = x * chunk + (bid >> 3), nblk >> 3, (x + 1) * chunk
        else: q, step, end = bid, nblk, ntiles
        while q < end:
            seen[q] += 1; q += step
    assert all(v == 1 for v in seen)
    wbuf = pl["mtiles"] * 4 * pl["nchunks"] * KK * 64 * 2          # doubles written by cpd::wimg_kernel = the workspace asked for
    xsize, ysize = B * C * H * W, B * M * L
    for q in sorted({0, 1, pl["tpi"] - 1, pl["tpi"], bt - 1, ntiles - 1, ntiles // 2} & set(range(ntiles))):
        mt, rem = divmod(q, bt); b, t = divmod(rem, pl["tpi"])
        pix0 = t * NPIX; py0 = pix0 // OW; iy_base = py0 * sh - ph; m0 = mt * 64
        for wave in range(4):
            for ch in (0, pl["nchunks"] - 1):
                a = ((mt * 4 + wave) * pl["nchunks"] + ch) * KK * 128 + 8 * 128 + 63 * 2
                assert a + 2 <= wbuf and a % 2 == 0, ("A", a, wbuf)
        for ch in (0, pl["nchunks"] - 1):
            for tid in range(NT):
                pq, xc = tid & 31, tid >> 5
                lane_in = pq < ((W + 1) >> 1); xcol = min(2 * pq, W - 2)
                for u in range(D_NXP):
                    iy = iy_base + u
                    if u < pl["PR"] and 0 <= iy < H:
                        a = ((b * C + ch * CC) * H + iy) * W + ((xc * H * W + xcol) if lane_in else 0)
                        assert 0 <= a and a + 2 <= xsize and a % 2 == 0, ("x", a, xsize)
                    if u < pl["PR"] and lane_in:
                        d = xc * PLANE + pw + xcol + u * PW
                        assert 0 <= d and d + 2 <= CC * PLANE, ("park", d)
        for pi in range(pix0, pix0 + NPIX):
            if pi >= L: continue
            py, px = divmod(pi, OW)
            off = (py - py0) * sh * PW + px * sw + 7 * PLANE + 2 * PW + 2   # last channel, last tap
            assert 0 <= (py - py0) * sh + 2 < pl["PR"] and px * sw + 2 < PW and off < CC * PLANE, ("B read", off)
            assert (b * M + min(M, m0 + 64) - 1) * L + pi < ysize
    return "f64 x%d ok" % pl["TN"]


F64_SHAPES = [  # B, C, H, W, M, (sh, sw), (ph, pw)
    (2, 64, 56, 56, 128, (1, 1), (1, 1)), (128, 64, 56, 56, 128, (1, 1), (1, 1)), (2, 8, 6, 12, 60, (1, 1), (1, 1)), (3, 16, 8, 36, 120, (1, 1), (0, 0)),
    (2, 24, 10, 16, 104, (1, 1), (2, 2)), (1, 8, 64, 64, 52, (1, 1), (1, 1)), (2, 16, 9, 62, 60, (2, 1), (1, 1)), (4, 32, 32, 32, 64, (1, 1), (1, 1)),
    (2, 8, 9, 64, 128, (2, 1), (1, 1)), (3, 8, 14, 28, 64, (1, 1), (1, 1)), (2, 8, 9, 30, 128, (1, 1), (0, 0)), (2, 32, 28, 28, 33, (1, 1), (1, 1)),
]


@pytest.mark.parametrize("case", F64_SHAPES, ids=str)
def test_f64_patch_kernel_loads_stay_inside_the_tensors(case):
    B, C, H, W, M, st, pd = case
    OH, OW = (H + 2 * pd[0] - 3) // st[0] + 1, (W + 2 * pd[1] - 3) // st[1] + 1
    plans = f64_plans(B, C, H, W, M, OH, OW, 3, 3, st[0], st[1], pd[0], pd[1])
    assert plans, "the shape must exercise the f64 patch kernel"
    for pl in plans:
        f64_walk(pl, min(B, 3), C, H, W, M, OH, OW, st[0], st[1], pd[0], pd[1])
    if st == (1, 1) and M % CC == 0 and OW % 2 == 0:  # the data gradient: a forward pass over grad_out, channels swapped, padding 2 - p
        for pl in f64_plans(B, M, OH, OW, C, H, W, 3, 3, 1, 1, 2 - pd[0], 2 - pd[1]):
            f64_walk(pl, min(B, 3), M, OH, OW, C, H, W, 1, 1, 2 - pd[0], 2 - pd[1])


# ---- wgrad_patch_f64.hpp: the f64 weight gradient -------------------------------------------------------------------------------
def wgd_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow, num_cus=256):
    if (kh != 3 or kw != 3 or sw != 1 or sh > 8 or Cin % 16 or Cout % 64 or W % 2 or W > 64 or ow % 8 or ow < 24 or ow > 64
            or ow // 8 not in (3, 4, 7, 8)): return None
    PW = W + 2 * pw; PLANE = (3 * PW) | 1; GP = ow | 1
    smem = max((64 * GP + 16 * PLANE + 16) * 8, 2 * 4 * 64 * 8)
    if smem > 72 * 1024: return None
    stages = B * oh; tiles = (Cin // 16) * (Cout // 64)
    splits = max(1, min(num_cus * 2 // tiles, max(1, stages // 4)))
    sps = _ceil_div(stages, splits)
    return dict(PW=PW, PLANE=PLANE, GP=GP, NK=ow // 8, stages=stages, sps=sps, splits=_ceil_div(stages, sps), smem=smem)
def wgd_walk(pl, B, Cin, H, W, Cout, sh, ph, pw, oh, ow):
    L, PW, PLANE, GP, NK = oh * ow, pl["PW"], pl["PLANE"], pl["GP"], pl["NK"]
    gsize, xsize = B * Cout * L, B * Cin * H * W
    covered = set()
    for z in range(pl["splits"]):
        covered |= set(range(z * pl["sps"], min(pl["stages"], (z + 1) * pl["sps"])))
    assert covered == set(range(pl["stages"]))
    assert PW == ow + 2 and PLANE >= 3 * PW and GP >= ow
    for s in (0, 1, oh - 1, oh, pl["stages"] - 1):
        if not 0 <= s < pl["stages"]: continue
        b, oy = divmod(s, oh); iy0 = oy * sh - ph
        for c0 in (0, Cin - 16):
            for oc0 in (0, Cout - 64):
                for tid in range(NT):
                    pq, prow = tid & 31, tid >> 5
                    if pq < ow // 2:
                        for u in range(8):
                            a = ((b * Cout + oc0 + prow + 8 * u) * L) + oy * ow + 2 * pq
                            assert 0 <= a and a + 2 <= gsize and a % 2 == 0, ("g", a)
                            d = (prow + 8 * u) * GP + 2 * pq
                            assert d + 2 <= 64 * GP
                    if pq < W // 2:
                        for r in range(3):
                            iy = iy0 + r
                            for cu in range(2):
                                if 0 <= iy < H:
                                    a = ((b * Cin + c0 + prow + 8 * cu) * H + iy) * W + 2 * pq
                                    assert 0 <= a and a + 2 <= xsize and a % 2 == 0, ("x", a)
                                d = (prow + 8 * cu) * PLANE + r * PW + pw + 2 * pq
                                assert d + 2 <= 16 * PLANE
    for wk in range(2):   # operand reads of the last pixel group
        pix = wk * 4 * NK + 4 * (NK - 1) + 3
        assert pix < ow and 63 * GP + pix < 64 * GP and 15 * PLANE + 2 * PW + pix + 2 < 16 * PLANE
    assert pl["splits"] * Cout * Cin * 9 * 8 > 0
    return "wgd ok"


WGD_SHAPES = [  # B, Cin, H, W, Cout, sh, (ph, pw)
    (128, 64, 56, 56, 128, 1, (1, 1)), (3, 16, 32, 32, 64, 1, (1, 1)), (2, 32, 26, 26, 64, 1, (0, 0)), (2, 16, 24, 62, 128, 1, (2, 2)),
    (2, 48, 47, 24, 64, 2, (1, 1)), (5, 16, 8, 64, 64, 1, (1, 1)),
]


@pytest.mark.parametrize("case", WGD_SHAPES, ids=str)
def test_f64_weight_gradient_patch_kernel_loads_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout, sh, pd = case
    oh, ow = (H + 2 * pd[0] - 3) // sh + 1, W + 2 * pd[1] - 2
    B = min(B, 3)  # the first and the last images are the ones at the tensor ends
    pl = wgd_plan(B, Cin, H, W, Cout, 3, 3, sh, 1, pd[0], pd[1], oh, ow)
    assert pl is not None, "the shape must exercise the f64 weight-gradient patch kernel"
    wgd_walk(pl, B, Cin, H, W, Cout, sh, pd[0], pd[1], oh, ow)


# ---- f32 stride-2 weight gradient (wgrad_patch_s2.hpp) ----
WG2_INSTANCES = [(1, 16, 4), (2, 16, 4), (4, 16, 4), (1, 32, 2), (2, 32, 2), (4, 32, 2)]
def wg2_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow, num_cus=256):
    if kh != 3 or kw != 3 or sh != 2 or sw != 2 or pw != 1 or ph > 1 or W != 2 * ow or Cin % 32 or Cout % 32: return None
    wmo = 4 if Cout % 128 == 0 else 2 if Cout % 64 == 0 else 1
    pick = [(a, o, r) for (a, o, r) in WG2_INSTANCES if a == wmo and o == ow and oh % r == 0]
    if not pick: return None
    WMO, OW, R = pick[0]
    stages = B * (oh // R); tiles = (Cin // 32) * (Cout // (32 * WMO))
    splits = max(1, min(num_cus // tiles, max(1, stages // 2)))
    sps = _ceil_div(stages, splits)
    return dict(WMO=WMO, OW=OW, R=R, stages=stages, sps=sps, splits=_ceil_div(stages, sps))
def wg2_walk(pl, B, Cin, H, Cout, ph, oh):
    WMO, OW, R = pl["WMO"], pl["OW"], pl["R"]
    WK, BM, W, PW, XR, KST = 4 // WMO, 32 * WMO, 2 * OW, 2 * OW + 2, 2 * R + 1, R * OW
    GP, PLANE = _odd_pitch_w(KST), _odd_pitch_w(XR * PW)
    XL = 8 if W <= 32 else 16
    RX = NT // XL; NXP = XR * 32 // RX; NG = BM // 16
    SEG = OW // WK; PAIRS = SEG // 2; BUF = BM * GP + 32 * PLANE
    red = 4 * (9 - 9 // WK) * 16 * 64 * 4 if WK == 2 else 4 * 16 * 64 * 4   # the closing sum's LDS slots
    assert XR * 32 % RX == 0 and max(2 * BUF * 4, red) <= 160 * 1024 and SEG % 2 == 0 and KST % 4 == 0 and KST <= 64
    L, spi = oh * OW, oh // R
    gsize, xsize = B * Cout * L, B * Cin * H * W
    covered = set()
    for z in range(pl["splits"]):
        covered |= set(range(z * pl["sps"], min(pl["stages"], (z + 1) * pl["sps"])))
    assert covered == set(range(pl["stages"]))
    rows_parked = set()
    for s in (0, 1, spi - 1, spi, pl["stages"] - 1):
        if not 0 <= s < pl["stages"]: continue
        b, k = divmod(s, spi); oy0 = k * R; iy0 = 2 * oy0 - ph
        for c0 in (0, Cin - 32):
            for oc0 in (0, Cout - BM):
                for tid in range(NT):
                    gq, grow, xq, xrow = tid & 15, tid >> 4, tid & (XL - 1), tid // XL
                    g_lane, x_lane = gq < KST // 4, xq < W // 4
                    for u in range(NG):
                        a = (b * Cout + oc0 + 16 * u + grow) * L + oy0 * OW + (4 * gq if g_lane else 0)
                        assert 0 <= a and a + 4 <= gsize and a % 4 == 0, ("g", a)
                        if g_lane:
                            d = (16 * u + grow) * GP + 4 * gq
                            assert d + 4 <= BM * GP
                    for u in range(NXP):
                        r, cb = u * RX // 32, u * RX % 32
                        iy = iy0 + r
                        assert cb + xrow < 32 and r < XR
                        if 0 <= iy < H:
                            a = ((b * Cin + c0 + cb + xrow) * H + iy) * W + (4 * xq if x_lane else 0)
                            assert 0 <= a and a + 4 <= xsize and a % 4 == 0, ("x", a)
                        if x_lane:
                            d = BM * GP + (cb + xrow) * PLANE + r * PW + 1 + 4 * xq
                            assert BM * GP <= d and d + 4 <= BUF
                            rows_parked.add((cb + xrow, r))
    assert rows_parked == {(c, r) for c in range(32) for r in range(XR)}
    # operand reads of every lane over the unrolled pixel loop stay inside the stage buffer, and the patch columns they touch are
    # columns 0 .. W: the zero column on the left and the W staged ones
    for wave in range(4):
        wmo, wk = wave % WMO, wave // WMO
        for lane in (0, 31, 32, 63):
            half, l32 = lane >> 5, lane & 31
            ga0 = (wmo * 32 + l32) * GP + wk * SEG + half
            xb0 = BM * GP + l32 * PLANE + 2 * (wk * SEG + half)
            for r in range(R):
                for j in range(PAIRS):
                    a = ga0 + r * OW + 2 * j
                    assert a - (wmo * 32 + l32) * GP < KST
                    for ky in range(3):
                        for kx in range(3):
                            d = xb0 + (2 * r + ky) * PW + 4 * j + kx
                            col = d - BM * GP - l32 * PLANE - (2 * r + ky) * PW
                            assert 0 <= col <= W and d < BUF
    return "wg2 ok"


WG2_SHAPES = [  # B, Cin, H, W, Cout, (ph, pw)
    (256, 32, 32, 32, 64, (1, 1)), (2, 64, 8, 32, 128, (1, 1)), (5, 32, 16, 32, 32, (1, 1)), (2, 32, 8, 64, 64, (1, 1)), (2, 64, 4, 64, 128, (1, 1)),
    (3, 32, 12, 64, 96, (1, 1)), (2, 32, 9, 32, 64, (0, 1)), (2, 32, 15, 32, 64, (1, 1)), (40, 32, 8, 32, 64, (1, 1)),
]


@pytest.mark.parametrize("case", WG2_SHAPES, ids=str)
def test_stride2_weight_gradient_patch_kernel_loads_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout, pd = case
    oh, ow = (H + 2 * pd[0] - 3) // 2 + 1, (W + 2 * pd[1] - 3) // 2 + 1
    B = min(B, 3)
    pl = wg2_plan(B, Cin, H, W, Cout, 3, 3, 2, 2, pd[0], pd[1], oh, ow)
    assert pl is not None, "the shape must exercise the stride-2 weight-gradient patch kernel"
    assert wg2_walk(pl, B, Cin, H, Cout, pd[0], oh) == "wg2 ok"


# ---- f32 stride-2 data gradient (dgrad_patch_s2.hpp) ----
DG2_INSTANCES = [(16, 16), (32, 16)]
def dg2_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow):
    if kh != 3 or kw != 3 or sh != 2 or sw != 2 or ph != 1 or pw != 1 or W != 2 * ow or H != 2 * oh or Cin % 32: return None
    pick = [(o, c) for (o, c) in DG2_INSTANCES if ow == o and Cout % c == 0 and oh % (256 // o) == 0]
    return dict(OW=pick[0][0], OCC=pick[0][1]) if pick else None
def dg2_walk(pl, B, Cin, Cout, oh):
    OW, OCC = pl["OW"], pl["OCC"]
    NTD, TR, PC = 512, 256 // OW, OW + 1
    PR = TR + 1; GPL = (PR * PC) | 1; KS = OCC // 2
    WCH, GCH = KS * 9 * 64, OCC * GPL; BUF = WCH + GCH
    W4 = OCC * 72; NWP = _ceil_div(W4, NTD); NGP = OCC * 64 // NTD; X4 = OCC * OW // 4
    assert 2 * BUF * 4 <= 160 * 1024 and OCC * 64 % NTD == 0 and X4 <= NTD
    L, H, W, tpi, nct = oh * OW, 2 * oh, 2 * OW, oh // TR, Cin // 32
    gsize, wsize, xsize = B * Cout * L, Cout * Cin * 9, B * Cin * H * W
    w_written, g_written = set(), set()
    for blk in sorted({0, 1, nct - 1, nct, B * tpi * nct - 1}):
        if not 0 <= blk < B * tpi * nct: continue
        bt, ct = divmod(blk, nct); b, tile = divmod(bt, tpi)
        c0, i0 = ct * 32, tile * TR
        next_row = i0 + TR < oh
        for k in (0, Cout // OCC - 1):
            oc0 = k * OCC
            first = blk == 0 and k == 0
            for tid in range(NTD):
                for u in range(NWP):
                    f = u * NTD + tid
                    ok = f < W4
                    ocl, q = divmod(f, 72)
                    a = c0 * 9 + oc0 * Cin * 9 + ((ocl * Cin * 9 + 4 * q) if ok else 0)
                    assert 0 <= a and a + 4 <= wsize and a % 4 == 0, ("w", a)
                    if ok and first:
                        for i in range(4):
                            c, t = divmod(4 * q + i, 9)
                            d = ((ocl >> 1) * 9 + t) * 64 + (ocl & 1) * 32 + c
                            assert 0 <= d < WCH
                            w_written.add(d)
                gq, goc = tid & 63, tid >> 6
                for u in range(NGP):
                    a = (b * Cout * oh + i0) * OW + (oc0 + 8 * u + goc) * L + 4 * gq
                    assert 0 <= a and a + 4 <= gsize and a % 4 == 0, ("g", a)
                    d = (8 * u + goc) * GPL + (gq // (OW // 4)) * PC + (gq % (OW // 4)) * 4
                    assert d + 4 <= GCH
                    if first: g_written.update(range(d, d + 4))
                xoc, xq = divmod(tid, OW // 4)
                if next_row:
                    a = (b * Cout * oh + i0) * OW + oc0 * L + ((xoc * L + TR * OW + 4 * xq) if tid < X4 else 0)
                    assert 0 <= a and a + 4 <= gsize and a % 4 == 0, ("g row", a)
                if tid < X4:
                    d = xoc * GPL + TR * PC + 4 * xq
                    assert d + 4 <= GCH
                    if first: g_written.update(range(d, d + 4))
        # stores: the pair of lane (cell, half) for accumulator element e and row class py
        for wave in range(8):
            for lane in (0, 15, 16, 31, 32, 63):
                half, l32 = lane >> 5, lane & 31
                crow, ccol = divmod(wave * 32 + l32, OW)
                for e in (0, 15):
                    c = 8 * (e >> 2) + 4 * half + (e & 3)
                    for py in range(2):
                        a = (((b * Cin + c0 + c) * H) + 2 * (i0 + crow) + py) * W + 2 * ccol
                        assert 0 <= a and a + 2 <= xsize and a % 2 == 0
                # operand reads: plane of oc = 2 ks + half, rows crow .. crow + 1, columns ccol .. ccol + 1
                for ks in (0, KS - 1):
                    d = (2 * ks + half) * GPL + (crow + 1) * PC + ccol + 1
                    assert d < GCH and crow + 1 < PR and ccol + 1 < PC
    assert w_written == set(range(WCH))
    # every patch element that the MFMA loop reads is staged or zeroed: all rows 0 .. TR, columns 0 .. OW - 1 staged, column OW zeroed
    need = {oc * GPL + r * PC + c for oc in range(OCC) for r in range(PR) for c in range(OW)}
    assert need <= g_written
    return "dg2 ok"


DG2_SHAPES = [  # B, Cin, H, W, Cout
    (256, 32, 32, 32, 64), (2, 64, 32, 32, 128), (2, 32, 64, 64, 32), (2, 64, 16, 64, 64), (2, 32, 32, 32, 48), (1, 96, 64, 32, 16),
]


@pytest.mark.parametrize("case", DG2_SHAPES, ids=str)
def test_stride2_data_gradient_patch_kernel_accesses_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout = case
    oh, ow = H // 2, W // 2
    B = min(B, 3)
    pl = dg2_plan(B, Cin, H, W, Cout, 3, 3, 2, 2, 1, 1, oh, ow)
    assert pl is not None, "the shape must exercise the stride-2 data-gradient patch kernel"
    assert dg2_walk(pl, B, Cin, Cout, oh) == "dg2 ok"


# ---- f64 stride-2 data gradient (dgrad_patch_s2_f64.hpp) ----
DGD2_INSTANCES = [(16, 8), (32, 8)]
def dgd2_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow):
    if kh != 3 or kw != 3 or sh != 2 or sw != 2 or ph != 1 or pw != 1 or W != 2 * ow or H != 2 * oh or Cin % 32: return None
    pick = [(o, c) for (o, c) in DGD2_INSTANCES if ow == o and Cout % c == 0 and oh % (256 // o) == 0]
    return dict(OW=pick[0][0], OCC=pick[0][1]) if pick else None
def dgd2_walk(pl, B, Cin, Cout, oh):
    """Offsets in doubles; 16-byte loads and stores must sit on even offsets."""
    OW, OCC = pl["OW"], pl["OCC"]
    NTD, TR, PC = 512, 256 // OW, OW + 1
    PR = TR + 1; GPL = (PR * PC) | 1; KS = OCC // 4
    WCH, GCH = KS * 9 * 2 * 64, OCC * GPL; BUF = WCH + GCH
    W2 = OCC * 144; NWP = _ceil_div(W2, NTD); NGP = OCC * 128 // NTD; X2 = OCC * OW // 2
    assert 2 * BUF * 8 <= 160 * 1024 and OCC * 128 % NTD == 0 and X2 <= NTD
    L, H, W, tpi, nct = oh * OW, 2 * oh, 2 * OW, oh // TR, Cin // 32
    gsize, wsize, xsize = B * Cout * L, Cout * Cin * 9, B * Cin * H * W
    w_written, g_written = set(), set()
    for blk in sorted({0, 1, nct - 1, nct, B * tpi * nct - 1}):
        if not 0 <= blk < B * tpi * nct: continue
        bt, ct = divmod(blk, nct); b, tile = divmod(bt, tpi)
        c0, i0 = ct * 32, tile * TR
        next_row = i0 + TR < oh
        for k in sorted({0, Cout // OCC - 1}):
            oc0 = k * OCC
            first = blk == 0 and k == 0
            for tid in range(NTD):
                for u in range(NWP):
                    f = u * NTD + tid
                    ok = f < W2
                    ocl, q = divmod(f, 144)
                    a = c0 * 9 + oc0 * Cin * 9 + ((ocl * Cin * 9 + 2 * q) if ok else 0)
                    assert 0 <= a and a + 2 <= wsize and a % 2 == 0, ("w", a)
                    if ok and first:
                        for i in range(2):
                            c, t = divmod(2 * q + i, 9)
                            d = (((ocl >> 2) * 9 + t) * 2 + (c >> 4)) * 64 + (ocl & 3) * 16 + (c & 15)
                            assert 0 <= d < WCH and d not in w_written
                            w_written.add(d)
                gq, goc = tid & 127, tid >> 7
                for u in range(NGP):
                    a = (b * Cout * oh + i0) * OW + (oc0 + 4 * u + goc) * L + 2 * gq
                    assert 0 <= a and a + 2 <= gsize and a % 2 == 0, ("g", a)
                    d = (4 * u + goc) * GPL + (gq // (OW // 2)) * PC + (gq % (OW // 2)) * 2
                    assert d + 2 <= GCH
                    if first: g_written.update(range(d, d + 2))
                xoc, xq = divmod(tid, OW // 2)
                if next_row:
                    a = (b * Cout * oh + i0) * OW + oc0 * L + ((xoc * L + TR * OW + 2 * xq) if tid < X2 else 0)
                    assert 0 <= a and a + 2 <= gsize and a % 2 == 0, ("g row", a)
                if tid < X2:
                    d = xoc * GPL + TR * PC + 2 * xq
                    assert d + 2 <= GCH and xoc < OCC
                    if first: g_written.update(range(d, d + 2))
        # stores and operand reads of the corner lanes: lane l holds rows 4 e + l / 16 of a 16 x 16 block, column l % 16
        for wave in range(8):
            for lane in (0, 15, 16, 47, 48, 63):
                kq, l16 = lane >> 4, lane & 15
                for h in range(2):
                    crow, ccol = divmod(wave * 32 + 16 * h + l16, OW)
                    for ch in range(2):
                        for e in (0, 3):
                            c = 16 * ch + 4 * e + kq
                            for py in range(2):
                                a = (((b * Cin + c0 + c) * H) + 2 * (i0 + crow) + py) * W + 2 * ccol
                                assert 0 <= a and a + 2 <= xsize and a % 2 == 0 and c0 + c < Cin
                    for ks in (0, KS - 1):
                        d = (4 * ks + kq) * GPL + (crow + 1) * PC + ccol + 1
                        assert d < GCH and crow + 1 < PR and ccol + 1 < PC
                        for t in range(9):
                            for ch in range(2):
                                assert ((ks * 9 + t) * 2 + ch) * 64 + lane < WCH
    assert w_written == set(range(WCH))
    need = {oc * GPL + r * PC + c for oc in range(OCC) for r in range(PR) for c in range(OW)}
    assert need <= g_written
    return "dgd2 ok"

DGD2_SHAPES = [  # B, Cin, H, W, Cout
    (256, 32, 32, 32, 64), (2, 64, 32, 32, 128), (2, 32, 64, 64, 32), (2, 64, 16, 64, 64), (2, 32, 32, 32, 8), (1, 96, 64, 32, 24),
]


@pytest.mark.parametrize("case", DGD2_SHAPES, ids=str)
def test_stride2_f64_data_gradient_patch_kernel_accesses_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout = case
    oh, ow = H // 2, W // 2
    B = min(B, 3)
    pl = dgd2_plan(B, Cin, H, W, Cout, 3, 3, 2, 2, 1, 1, oh, ow)
    assert pl is not None, "the shape must exercise the f64 stride-2 data-gradient patch kernel"
    assert dgd2_walk(pl, B, Cin, Cout, oh) == "dgd2 ok"


# ---- f64 stride-2 weight gradient (wgrad_patch_s2_f64.hpp) ----
WGD2_INSTANCES = [(16, 2), (32, 1)]
def wgd2_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow, num_cus=256):
    if kh != 3 or kw != 3 or sh != 2 or sw != 2 or pw != 1 or ph > 1 or W != 2 * ow or Cin % 32 or Cout % 64: return None
    pick = [(o, r) for (o, r) in WGD2_INSTANCES if o == ow and oh % r == 0]
    if not pick: return None
    OW, R = pick[0]
    stages = B * (oh // R); tiles = (Cin // 32) * (Cout // 64)
    splits = max(1, min(num_cus // tiles, max(1, stages // 2)))
    sps = _ceil_div(stages, splits)
    return dict(OW=OW, R=R, stages=stages, sps=sps, splits=_ceil_div(stages, sps))
def wgd2_walk(pl, B, Cin, H, Cout, ph, oh):
    """Offsets in doubles; 16-byte loads must sit on even offsets."""
    OW, R = pl["OW"], pl["R"]
    NTW, BM, W, PW, XR, KST = 256, 64, 2 * OW, 2 * OW + 2, 2 * R + 1, R * OW
    GP, PLANE = KST | 1, (XR * PW) | 1
    XL, GL = W // 2, KST // 2
    RX, GR = NTW // XL, NTW // GL
    NXP, NG = XR * 32 // RX, BM // GR
    GROUPS, GPR, BUF = KST // 4, OW // 4, BM * GP + 32 * PLANE
    assert NTW % XL == 0 and 32 % RX == 0 and NTW % GL == 0 and BM % GR == 0 and 2 * BUF * 8 <= 160 * 1024
    L, spi = oh * OW, oh // R
    gsize, xsize = B * Cout * L, B * Cin * H * W
    covered = set()
    for z in range(pl["splits"]):
        covered |= set(range(z * pl["sps"], min(pl["stages"], (z + 1) * pl["sps"])))
    assert covered == set(range(pl["stages"]))
    rows_parked, g_parked = set(), set()
    for s in (0, 1, spi - 1, spi, pl["stages"] - 1):
        if not 0 <= s < pl["stages"]: continue
        b, k = divmod(s, spi); oy0 = k * R; iy0 = 2 * oy0 - ph
        for c0 in (0, Cin - 32):
            for oc0 in (0, Cout - BM):
                for tid in range(NTW):
                    gq, grow, xq, xrow = tid % GL, tid // GL, tid % XL, tid // XL
                    for u in range(NG):
                        a = (b * Cout + oc0 + GR * u + grow) * L + oy0 * OW + 2 * gq
                        assert 0 <= a and a + 2 <= gsize and a % 2 == 0, ("g", a)
                        d = (GR * u + grow) * GP + 2 * gq
                        assert d + 2 <= BM * GP and 2 * gq + 2 <= KST
                        g_parked.update((GR * u + grow, 2 * gq + i) for i in range(2))
                    for u in range(NXP):
                        r, cb = u * RX // 32, u * RX % 32
                        iy = iy0 + r
                        assert cb + xrow < 32 and r < XR
                        if 0 <= iy < H:
                            a = ((b * Cin + c0 + cb + xrow) * H + iy) * W + 2 * xq
                            assert 0 <= a and a + 2 <= xsize and a % 2 == 0, ("x", a)
                        d = BM * GP + (cb + xrow) * PLANE + r * PW + 1 + 2 * xq
                        assert BM * GP <= d and d + 2 <= BUF and 1 + 2 * xq + 2 <= W + 1
                        rows_parked.update((cb + xrow, r, 1 + 2 * xq + i) for i in range(2))
    assert rows_parked == {(c, r, col) for c in range(32) for r in range(XR) for col in range(1, W + 1)}
    assert g_parked == {(oc, px) for oc in range(BM) for px in range(KST)}
    # operand reads of the corner lanes over the unrolled pixel loop: pixels inside the stage, patch columns 0 .. W
    for wave in range(4):
        wmo, wc = wave & 1, wave >> 1
        for lane in (0, 15, 16, 47, 48, 63):
            kq, l16 = lane >> 4, lane & 15
            ga0 = (wmo * 32 + l16) * GP + kq
            xb0 = BM * GP + (wc * 16 + l16) * PLANE + 2 * kq
            for u in range(GROUPS):
                r, j = divmod(u, GPR)
                for o in range(2):
                    a = ga0 + 16 * o * GP + r * OW + 4 * j
                    assert a - (wmo * 32 + 16 * o + l16) * GP < KST and a < BM * GP
                for ky in range(3):
                    for kx in range(3):
                        d = xb0 + (2 * r + ky) * PW + 8 * j + kx
                        col = d - BM * GP - (wc * 16 + l16) * PLANE - (2 * r + ky) * PW
                        assert 0 <= col <= W and d < BUF and 2 * r + ky < XR
                        assert col == 2 * (4 * j + kq) + kx
            for o in range(2):
                for e in (0, 3):
                    oc = wmo * 32 + o * 16 + 4 * e + kq
                    assert oc < BM and wc * 16 + l16 < 32
    return "wgd2 ok"

WGD2_SHAPES = [  # B, Cin, H, W, Cout, (ph, pw)
    (256, 32, 32, 32, 64, (1, 1)), (2, 64, 8, 32, 128, (1, 1)), (2, 32, 8, 64, 64, (1, 1)), (2, 64, 4, 64, 128, (1, 1)),
    (2, 32, 33, 32, 64, (0, 1)), (2, 32, 31, 32, 64, (1, 1)), (40, 32, 8, 32, 64, (1, 1)), (3, 32, 6, 64, 192, (1, 1)),
]


@pytest.mark.parametrize("case", WGD2_SHAPES, ids=str)
def test_stride2_f64_weight_gradient_patch_kernel_accesses_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout, pd = case
    oh, ow = (H + 2 * pd[0] - 3) // 2 + 1, (W + 2 * pd[1] - 3) // 2 + 1
    B = min(B, 41)
    pl = wgd2_plan(B, Cin, H, W, Cout, 3, 3, 2, 2, pd[0], pd[1], oh, ow)
    assert pl is not None, "the shape must exercise the f64 stride-2 weight-gradient patch kernel"
    assert wgd2_walk(pl, B, Cin, H, Cout, pd[0], oh) == "wgd2 ok"


# ---- f32 stride-2 forward pass (fwd_patch_s2.hpp) ----
FW2_INSTANCES = [(16, 2), (16, 1), (32, 2), (32, 1)]
def fw2_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow):
    if kh != 3 or kw != 3 or sh != 2 or sw != 2 or ph != 1 or pw != 1 or W != 2 * ow or H != 2 * oh or Cin % 8 or Cout % 32: return None
    if not (Cout == 32 or (Cout == 64 and Cin <= 16)): return None
    mb = 2 if Cout % 64 == 0 else 1
    pick = [(o, m) for (o, m) in FW2_INSTANCES if ow == o and mb == m and oh % (256 // o) == 0]
    return dict(OW=pick[0][0], MB=pick[0][1]) if pick else None
def fw2_walk(pl, B, Cin, Cout, oh):
    OW, MB = pl["OW"], pl["MB"]
    NTF, CC, TR, HALF = 512, 8, 256 // OW, OW + 1
    PR, W, H = 2 * TR + 1, 2 * OW, 2 * oh
    RP = 40 if OW == 16 else 2 * HALF
    PLANE = (PR * RP) | 1
    WCH, XCH = (CC // 2) * 9 * MB * 64, CC * PLANE; BUF = WCH + XCH
    W4, X4 = MB * 32 * CC * 9 // 4, CC * PR * (W // 4)
    NWP, NXP = _ceil_div(W4, NTF), _ceil_div(X4, NTF)
    assert 2 * BUF * 4 <= 160 * 1024 and 2 * HALF <= RP
    L, tpi, nmt = oh * OW, oh // TR, Cout // (32 * MB)
    xsize, wsize, ysize = B * Cin * H * W, Cout * Cin * 9, B * Cout * L
    nblk = B * tpi * nmt
    w_written, x_written = set(), set()
    for blk in sorted({0, 1, nmt - 1, nmt, nblk - 1}):
        if not 0 <= blk < nblk: continue
        bt, mt = divmod(blk, nmt); b, tile = divmod(bt, tpi)
        oc0, oy0 = mt * 32 * MB, tile * TR
        iy0 = 2 * oy0 - 1
        for k in sorted({0, Cin // CC - 1}):
            c0 = k * CC
            first = blk == 0 and k == 0
            for tid in range(NTF):
                for u in range(NWP):
                    f = u * NTF + tid
                    ok = f < W4
                    ocl, q = divmod(f, 18)
                    a = oc0 * Cin * 9 + c0 * 9 + ((ocl * Cin * 9 + 4 * q) if ok else 0)
                    assert 0 <= a and a + 4 <= wsize and a % 4 == 0, ("w", a)
                    if ok and first:
                        for i in range(4):
                            cl, t = divmod(4 * q + i, 9)
                            d = (((cl >> 1) * 9 + t) * MB + (ocl >> 5)) * 64 + (cl & 1) * 32 + (ocl & 31)
                            assert 0 <= d < WCH and d not in w_written
                            w_written.add(d)
                for u in range(NXP):
                    f = u * NTF + tid
                    inside = f < X4
                    cr, q = divmod(f, W // 4); c, r = divmod(cr, PR)
                    iy = iy0 + r
                    ok = inside and 0 <= iy < H
                    a = b * Cin * H * W + c0 * H * W + (((c * H + iy) * W + 4 * q) if ok else 0)
                    assert 0 <= a and a + 4 <= xsize and a % 4 == 0, ("x", a)
                    if inside:
                        d = c * PLANE + r * RP + 2 * q
                        for o in (HALF, 1, HALF + 1, 2):
                            assert 0 <= d + o < XCH and (not first or d + o not in x_written)
                            if first: x_written.add(d + o)
        # the zero column, operand reads and stores of the corner lanes
        if blk == 0:
            for i in range(2 * CC * PR):
                buf, rem = divmod(i, CC * PR); c, r = divmod(rem, PR)
                assert buf < 2
                d = c * PLANE + r * RP
                assert d not in x_written or buf == 1
                if buf == 0: x_written.add(d)
        for wave in range(8):
            for lane in (0, 15, 16, 31, 32, 47, 63):
                half, l32 = lane >> 5, lane & 31
                pix = wave * 32 + l32
                prow, pcol = divmod(pix, OW)
                for cp in (0, CC // 2 - 1):
                    for t in range(9):
                        ky, kx = divmod(t, 3)
                        d = (half + 2 * cp) * PLANE + (2 * prow + ky) * RP + pcol + (HALF if kx == 1 else 0) + (1 if kx == 2 else 0)
                        # the word holds patch row 2 prow + ky, patch column 2 pcol + kx of channel 2 cp + half
                        c, rem = divmod(d, PLANE); r, o = divmod(rem, RP)
                        assert c == 2 * cp + half and r == 2 * prow + ky and r < PR
                        pc = 2 * o if o < HALF else 2 * (o - HALF) + 1
                        assert o < 2 * HALF and pc == 2 * pcol + kx
                        assert blk != 0 or d in x_written
                        for m in range(MB):
                            assert ((cp * 9 + t) * MB + m) * 64 + lane < WCH
                for m in range(MB):
                    for e in (0, 15):
                        oc = m * 32 + 8 * (e >> 2) + 4 * half + (e & 3)
                        a = (b * Cout + oc0 + oc) * L + oy0 * OW + pix
                        assert 0 <= a < ysize and oc0 + oc < Cout and oy0 * OW + pix < L
    assert w_written == set(range(WCH))
    return "fw2 ok"

FW2_SHAPES = [  # B, Cin, H, W, Cout
    (256, 32, 32, 32, 32), (2, 8, 32, 32, 32), (2, 16, 64, 64, 64), (2, 24, 16, 64, 32), (3, 40, 64, 32, 32), (2, 8, 32, 32, 64),
]


@pytest.mark.parametrize("case", FW2_SHAPES, ids=str)
def test_stride2_forward_patch_kernel_accesses_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout = case
    oh, ow = H // 2, W // 2
    B = min(B, 3)
    pl = fw2_plan(B, Cin, H, W, Cout, 3, 3, 2, 2, 1, 1, oh, ow)
    assert pl is not None, "the shape must exercise the stride-2 forward patch kernel"
    assert fw2_walk(pl, B, Cin, Cout, oh) == "fw2 ok"


# ---- f64 stride-2 forward pass (fwd_patch_s2_f64.hpp) ----
def fwd2_plan(B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow):
    if kh != 3 or kw != 3 or sh != 2 or sw != 2 or ph != 1 or pw != 1 or W != 2 * ow or H != 2 * oh or Cin % 4 or Cout not in (32, 64): return None
    mb = 2 if Cout % 64 == 0 else 1
    pick = [(o, m) for (o, m) in FW2_INSTANCES if ow == o and mb == m and oh % (256 // o) == 0]
    return dict(OW=pick[0][0], MB=pick[0][1]) if pick else None
def fwd2_walk(pl, B, Cin, Cout, oh):
    """Offsets in doubles; 16-byte loads must sit on even offsets."""
    OW, MB = pl["OW"], pl["MB"]
    NTF, CC, TR, HALF, NB = 512, 4, 256 // OW, OW + 1, 2 * MB
    PR, W, H = 2 * TR + 1, 2 * OW, 2 * oh
    RP = 40 if OW == 16 else 2 * HALF
    PLANE = (PR * RP) | 1
    WCH, XCH = 9 * NB * 64, CC * PLANE; BUF = WCH + XCH
    W2, X2 = MB * 32 * CC * 9 // 2, CC * PR * (W // 2)
    NWP, NXP = _ceil_div(W2, NTF), _ceil_div(X2, NTF)
    assert 2 * BUF * 8 <= 160 * 1024 and 2 * HALF <= RP
    L, tpi, nmt = oh * OW, oh // TR, Cout // (32 * MB)
    xsize, wsize, ysize = B * Cin * H * W, Cout * Cin * 9, B * Cout * L
    nblk = B * tpi * nmt
    w_written, x_written = set(), set()
    for blk in sorted({0, 1, nmt - 1, nmt, nblk - 1}):
        if not 0 <= blk < nblk: continue
        bt, mt = divmod(blk, nmt); b, tile = divmod(bt, tpi)
        oc0, oy0 = mt * 32 * MB, tile * TR
        iy0 = 2 * oy0 - 1
        for k in sorted({0, Cin // CC - 1}):
            c0 = k * CC
            first = blk == 0 and k == 0
            for tid in range(NTF):
                for u in range(NWP):
                    f = u * NTF + tid
                    ok = f < W2
                    ocl, q = divmod(f, 18)
                    a = oc0 * Cin * 9 + c0 * 9 + ((ocl * Cin * 9 + 2 * q) if ok else 0)
                    assert 0 <= a and a + 2 <= wsize and a % 2 == 0, ("w", a)
                    if ok and first:
                        for i in range(2):
                            cl, t = divmod(2 * q + i, 9)
                            d = (t * NB + (ocl >> 4)) * 64 + cl * 16 + (ocl & 15)
                            assert 0 <= d < WCH and d not in w_written
                            w_written.add(d)
                for u in range(NXP):
                    f = u * NTF + tid
                    inside = f < X2
                    cr, q = divmod(f, W // 2); c, r = divmod(cr, PR)
                    iy = iy0 + r
                    ok = inside and 0 <= iy < H
                    a = b * Cin * H * W + c0 * H * W + (((c * H + iy) * W + 2 * q) if ok else 0)
                    assert 0 <= a and a + 2 <= xsize and a % 2 == 0, ("x", a)
                    if inside:
                        d = c * PLANE + r * RP + q
                        for o in (HALF, 1):
                            assert 0 <= d + o < XCH and (not first or d + o not in x_written)
                            if first: x_written.add(d + o)
        if blk == 0:
            for i in range(2 * CC * PR):
                buf, rem = divmod(i, CC * PR); c, r = divmod(rem, PR)
                d = c * PLANE + r * RP
                assert buf < 2 and (d not in x_written or buf == 1)
                if buf == 0: x_written.add(d)
        for wave in range(8):
            for lane in (0, 15, 16, 47, 48, 63):
                kq, l16 = lane >> 4, lane & 15
                for h in range(2):
                    pix = wave * 32 + 16 * h + l16
                    prow, pcol = divmod(pix, OW)
                    for t in range(9):
                        ky, kx = divmod(t, 3)
                        d = kq * PLANE + (2 * prow + ky) * RP + pcol + (HALF if kx == 1 else 0) + (1 if kx == 2 else 0)
                        c, rem = divmod(d, PLANE); r, o = divmod(rem, RP)
                        assert c == kq and r == 2 * prow + ky and r < PR and o < 2 * HALF
                        pc = 2 * o if o < HALF else 2 * (o - HALF) + 1
                        assert pc == 2 * pcol + kx and (blk != 0 or d in x_written)
                        for m in range(NB):
                            assert (t * NB + m) * 64 + lane < WCH
                    for m in range(NB):
                        for e in (0, 3):
                            oc = 16 * m + 4 * e + kq
                            a = (b * Cout + oc0 + oc) * L + oy0 * OW + pix
                            assert 0 <= a < ysize and oc0 + oc < Cout and oy0 * OW + pix < L
    assert w_written == set(range(WCH))
    return "fwd2 ok"

FWD2_SHAPES = [  # B, Cin, H, W, Cout
    (256, 32, 32, 32, 64), (2, 4, 32, 32, 32), (2, 16, 64, 64, 64), (2, 12, 16, 64, 32), (3, 40, 64, 32, 64),
]


@pytest.mark.parametrize("case", FWD2_SHAPES, ids=str)
def test_stride2_f64_forward_patch_kernel_accesses_stay_inside_the_tensors(case):
    B, Cin, H, W, Cout = case
    oh, ow = H // 2, W // 2
    B = min(B, 3)
    pl = fwd2_plan(B, Cin, H, W, Cout, 3, 3, 2, 2, 1, 1, oh, ow)
    assert pl is not None, "the shape must exercise the f64 stride-2 forward patch kernel"
    assert fwd2_walk(pl, B, Cin, Cout, oh) == "fwd2 ok"


# ---- f64 image layer, forward and weight gradient (conv_image_f64.hpp) ----
def cim_walk(B, Cin, H, Cout, wgrad, num_cus=256):
    """Offsets in doubles; 16-byte loads must sit on even offsets."""
    NTI, W, TR, CP = 512, 32, 8, 4
    PR, PW = TR + 2, W + 2
    PLANE = (PR * PW) | 1
    X2 = CP * PR * (W // 2)
    L, K, tpi = H * W, Cin * 9, H // TR
    xsize, gsize = B * Cin * L, B * Cout * L
    assert H % TR == 0 and Cout % 32 == 0 and 1 <= Cin <= (3 if wgrad else 4) and X2 <= 2 * NTI
    tiles = B * tpi

    def stage_patch(b, oy0):
        cells = set()
        for f in range(X2):
            cr, q = divmod(f, W // 2); c, r = divmod(cr, PR)
            iy = oy0 - 1 + r
            if c < Cin and 0 <= iy < H:
                a = b * Cin * L + (c * H + iy) * W + 2 * q
                assert 0 <= a and a + 2 <= xsize and a % 2 == 0, ("x", a)
            d = c * PLANE + r * PW + 1 + 2 * q
            assert d + 2 <= CP * PLANE
            cells.update((d, d + 1))
        for i in range(CP * PR * 2):
            cr = i >> 1
            cells.add((cr // PR) * PLANE + (cr % PR) * PW + (i & 1) * (W + 1))
        return cells

    if not wgrad:
        nmt = Cout // 32
        for blk in sorted({0, nmt - 1, nmt, tiles * nmt - 1}):
            bt, mt = divmod(blk, nmt); b, tile = divmod(bt, tpi)
            oc0, oy0 = mt * 32, tile * TR
            cells = stage_patch(b, oy0)
            wcells = set()
            for i in range(32 * CP * 9):
                ocl, r = divmod(i, CP * 9); cl, t = divmod(r, 9)
                if cl < Cin: assert (oc0 + ocl) * K + cl * 9 + t < Cout * K
                wcells.add((t * 2 + (ocl >> 4)) * 64 + cl * 16 + (ocl & 15))
            assert wcells == set(range(9 * 2 * 64))
            for wave in range(8):
                for lane in (0, 15, 16, 63):
                    kq, l16 = lane >> 4, lane & 15
                    for h in range(2):
                        pix = wave * 32 + 16 * h + l16
                        for t in range(9):
                            d = kq * PLANE + (pix // W + t // 3) * PW + pix % W + t % 3
                            assert d in cells
                        for m in range(2):
                            for e in (0, 3):
                                a = (b * Cout + oc0 + 16 * m + 4 * e + kq) * L + oy0 * W + pix
                                assert 0 <= a < gsize
        return "cim fwd ok"
    rows = Cout // 32
    splits = max(1, min(2 * num_cus // rows, max(1, tiles // 2)))
    tps = _ceil_div(tiles, splits); splits = _ceil_div(tiles, tps)
    covered = set()
    for z in range(splits): covered |= set(range(z * tps, min(tiles, (z + 1) * tps)))
    assert covered == set(range(tiles))
    GP = 257
    assert (max(32 * GP + CP * PLANE, 8 * 16 * 64)) * 8 <= 96 * 1024
    for tl in sorted({0, tpi - 1, tiles - 1}):
        b, tile = divmod(tl, tpi); oy0 = tile * TR
        cells = stage_patch(b, oy0)
        for oc0 in (0, Cout - 32):
            gcells = set()
            for f in range(8 * NTI):
                row, q = f >> 7, f & 127
                a = (b * Cout + oc0 + row) * L + oy0 * W + 2 * q
                assert 0 <= a and a + 2 <= gsize and a % 2 == 0, ("g", a)
                gcells.update((row * GP + 2 * q, row * GP + 2 * q + 1))
            for wave in range(8):
                for lane in (0, 15, 16, 26, 63):
                    kq, l16 = lane >> 4, lane & 15
                    for s in range(W // 4):
                        for m in range(2):
                            assert (l16 + 16 * m) * GP + wave * W + kq + 4 * s in gcells
                        for nb in range(2):
                            kp = 16 * nb + l16
                            c, t = divmod(kp, 9) if kp < K else (0, 0)
                            d = c * PLANE + (wave + t // 3) * PW + t % 3 + kq + 4 * s
                            assert d in cells
                            # the word is pixel (row wave, column 4 s + kq) shifted by the tap
                            assert d == c * PLANE + (wave + t // 3) * PW + (4 * s + kq) + t % 3
    # partial sums: [splits][Cout][K], every (oc, pair < K) written once per split
    for z in (0, splits - 1):
        for oc0 in (0, Cout - 32):
            seen = set()
            for wave in range(8):
                for u in range(2):
                    el = 2 * wave + u; blk, e = el >> 2, el & 3
                    for lane in range(64):
                        kq, l16 = lane >> 4, lane & 15
                        oc, kp = 16 * (blk >> 1) + 4 * e + kq, 16 * (blk & 1) + l16
                        if kp < K:
                            a = (z * Cout + oc0 + oc) * K + kp
                            assert 0 <= a < splits * Cout * K and a not in seen
                            seen.add(a)
            assert len(seen) == 32 * K
    return "cim wgrad ok"


@pytest.mark.parametrize("case", [(256, 3, 32, 32), (2, 1, 8, 64), (3, 4, 40, 96), (5, 2, 24, 32)], ids=str)
def test_f64_image_layer_kernels_accesses_stay_inside_the_tensors(case):
    B, Cin, H, Cout = case
    B = min(B, 9)
    assert cim_walk(B, Cin, H, Cout, wgrad=False) == "cim fwd ok"
    if Cin <= 3:
        assert cim_walk(B, Cin, H, Cout, wgrad=True) == "cim wgrad ok"
