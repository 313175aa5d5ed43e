"""The reference's end-to-end tested tile programs, written against `KernelBuilder`.

These are input programs, not product logic: each is a statement-for-statement restatement of a Lean
`@[gpu_kernel]` definition (names and tile shapes included), because the task of the emitter is to run
those very programs on gfx950.  The product logic is the emitter and the tile library they are lowered by.

Each function builds the same statement sequence as the Lean definition it cites; together they
are the kernels the reference ships runners for (Examples/GPU/Run{Copy,Rotary,LayerNorm,FlashAttn}.lean)
plus its canonical GEMM example.
"""
from __future__ import annotations

from .builder import KernelBuilder
from .ir import Kernel


def copy64x64() -> Kernel:
    """Tyr/GPU/Kernels/Copy.lean:16-26 -- one 64x64 f32 tile, global -> LDS -> registers and back."""
    k = KernelBuilder("copy64x64")
    inp = k.gptr("Float32", "input")
    out = k.gptr("Float32", "output")
    k.comment("ThunderKittens-style minimal copy kernel")
    coord = k.blockCoord2D()
    reg = k.allocRT("Float32", 64, 64)
    smem = k.allocST("Float32", 64, 64)
    k.loadGlobal(smem, inp, coord)
    k.load(reg, smem)
    k.store(smem, reg)
    k.storeGlobal(out, smem, coord)
    k.sync()
    return k.build()


def rotaryFwd() -> Kernel:
    """Tyr/GPU/Kernels/Rotary.lean:13-62 -- RoPE on one 64x64 tile split as [x1 | x2]."""
    k = KernelBuilder("rotaryFwd")
    x_ptr = k.gptr("Float32", "x_ptr")
    sin_ptr = k.gptr("Float32", "sin_ptr")
    cos_ptr = k.gptr("Float32", "cos_ptr")
    out_ptr = k.gptr("Float32", "out_ptr")
    k.kval("UInt64", "_seq_len")
    k.kval("UInt64", "_head_dim")
    coord = k.blockCoord2D()

    x = k.allocRT("Float32", 64, 64)
    x1 = k.allocRT("Float32", 64, 32)
    x2 = k.allocRT("Float32", 64, 32)
    sinT = k.allocRT("Float32", 64, 32)
    cosT = k.allocRT("Float32", 64, 32)
    y1 = k.allocRT("Float32", 64, 32)
    y2 = k.allocRT("Float32", 64, 32)
    tmp = k.allocRT("Float32", 64, 32)
    negX2 = k.allocRT("Float32", 64, 32)
    out = k.allocRT("Float32", 64, 64)

    xShared = k.allocST("Float32", 64, 64)
    sinShared = k.allocST("Float32", 64, 32)
    cosShared = k.allocST("Float32", 64, 32)
    outShared = k.allocST("Float32", 64, 64)

    k.loadGlobal(xShared, x_ptr, coord)
    k.loadGlobal(sinShared, sin_ptr, coord)
    k.loadGlobal(cosShared, cos_ptr, coord)
    k.sync()

    k.load(x, xShared)
    k.load(sinT, sinShared)
    k.load(cosT, cosShared)

    k.sliceCols(x1, x, 0, 32)
    k.sliceCols(x2, x, 32, 32)

    # y1 = x1*cos - x2*sin
    k.mul(y1, x1, cosT)
    k.neg(negX2, x2)
    k.mul(negX2, negX2, sinT)
    k.add(y1, y1, negX2)

    # y2 = x2*cos + x1*sin
    k.mul(y2, x2, cosT)
    k.mul(tmp, x1, sinT)
    k.add(y2, y2, tmp)

    k.concatCols(out, y1, y2)

    k.store(outShared, out)
    k.sync()
    k.storeGlobal(out_ptr, outShared, coord)
    return k.build()


def tkFusedLayerNormResidual1024() -> Kernel:
    """Tyr/GPU/Kernels/FusedLayerNorm.lean:28-126 -- residual add + LayerNorm over d_model = 1024 on
    64-row blocks, two passes over sixteen 64x64 tiles."""
    k = KernelBuilder("tkFusedLayerNormResidual1024")
    x_ptr = k.gptr("BFloat16", "x_ptr")
    residual_ptr = k.gptr("BFloat16", "residual_ptr")
    weight_ptr = k.gptr("BFloat16", "weight_ptr")
    bias_ptr = k.gptr("BFloat16", "bias_ptr")
    out_ptr = k.gptr("BFloat16", "out_ptr")
    out_resid_ptr = k.gptr("BFloat16", "out_resid_ptr")
    k.comment("ThunderKittens-style layernorm + residual on 64x1024 tiles")

    hiddenTiles = 16
    invHidden = 0.0009765625
    eps = 1.0e-5

    coord = k.blockCoord2D()

    x = k.allocRT("BFloat16", 64, 64)
    residual = k.allocRT("BFloat16", 64, 64)
    outResid = k.allocRT("BFloat16", 64, 64)
    outResidF = k.allocRT("Float32", 64, 64)
    centered = k.allocRT("Float32", 64, 64)
    sq = k.allocRT("Float32", 64, 64)

    tileShared = k.allocST("BFloat16", 64, 64)

    sum_ = k.zeroRV("Float32", 64)
    sumSq = k.zeroRV("Float32", 64)
    tmpSum = k.allocRV("Float32", 64)
    tmpSqSum = k.allocRV("Float32", 64)
    mean = k.allocRV("Float32", 64)
    meanSq = k.allocRV("Float32", 64)
    var = k.allocRV("Float32", 64)
    invStd = k.allocRV("Float32", 64)

    weightShared = k.allocSV("BFloat16", 64)
    biasShared = k.allocSV("BFloat16", 64)
    weightRV = k.allocRV("BFloat16", 64)
    biasRV = k.allocRV("BFloat16", 64)
    weightF = k.allocRV("Float32", 64)
    biasF = k.allocRV("Float32", 64)

    k.comment("Pass 1: out_resid and row statistics across full hidden dimension")
    with k.krange(0, hiddenTiles) as hiddenIdx:
        tileCoord = coord.withCol(hiddenIdx.id)

        k.loadGlobal(tileShared, x_ptr, tileCoord)
        k.sync()
        k.load(x, tileShared)

        k.loadGlobal(tileShared, residual_ptr, tileCoord)
        k.sync()
        k.load(residual, tileShared)

        k.add(outResid, x, residual)
        k.store(tileShared, outResid)
        k.sync()
        k.storeGlobal(out_resid_ptr, tileShared, tileCoord)

        k.convert(outResidF, outResid)
        k.rowSum(tmpSum, outResidF)
        k.addVec(sum_, sum_, tmpSum)
        k.mul(sq, outResidF, outResidF)
        k.rowSum(tmpSqSum, sq)
        k.addVec(sumSq, sumSq, tmpSqSum)

    k.scalarMulVec(mean, sum_, invHidden)
    k.scalarMulVec(var, sumSq, invHidden)
    k.mulVec(meanSq, mean, mean)
    k.subVec(var, var, meanSq)
    k.scalarAddVec(var, var, eps)
    k.rsqrtVec(invStd, var)

    k.comment("Pass 2: normalize + affine (weight, bias)")
    with k.krange(0, hiddenTiles) as hiddenIdx:
        tileCoord = coord.withCol(hiddenIdx.id)

        k.loadGlobal(tileShared, out_resid_ptr, tileCoord)
        k.sync()
        k.load(outResid, tileShared)
        k.convert(outResidF, outResid)

        k.loadVecGlobalCol(weightShared, weight_ptr, tileCoord)
        k.loadVec(weightRV, weightShared)
        k.convertVec(weightF, weightRV)

        k.loadVecGlobalCol(biasShared, bias_ptr, tileCoord)
        k.loadVec(biasRV, biasShared)
        k.convertVec(biasF, biasRV)

        k.subCol(centered, outResidF, mean)
        k.mulCol(centered, centered, invStd)
        k.mulRow(centered, centered, weightF)
        k.addRow(centered, centered, biasF)

        k.convert(outResid, centered)
        k.store(tileShared, outResid)
        k.sync()
        k.storeGlobal(out_ptr, tileShared, tileCoord)
    return k.build()


def simpleGemm(numKBlocks: int = 8) -> Kernel:
    """Tyr/GPU/Kernels/Examples.lean:23-65 -- C[64x64 tile] = sum over numKBlocks of A tile x B tile,
    bf16 operands, f32 accumulator and output."""
    k = KernelBuilder("simpleGemm")
    aPtr = k.gptr("BFloat16", "aPtr")
    bPtr = k.gptr("BFloat16", "bPtr")
    cPtr = k.gptr("Float32", "cPtr")
    k.kval("UInt64", "m")
    k.kval("UInt64", "n")
    k.kval("UInt64", "k")
    k.comment("=== Example GEMM ===")
    coord = k.blockCoord2D()

    a = k.allocRT("BFloat16", 64, 64)
    b = k.allocRT("BFloat16", 64, 64, "Col")
    c = k.zeroRT("Float32", 64, 64)

    aS = k.allocST("BFloat16", 64, 64)
    bS = k.allocST("BFloat16", 64, 64, "Col")
    cS = k.allocST("Float32", 64, 64)

    with k.krange(0, numKBlocks) as kBlk:
        k.loadGlobal(aS, aPtr, coord.withCol(kBlk.id))
        k.loadGlobal(bS, bPtr, coord.withRow(kBlk.id))
        k.sync()
        k.load(a, aS)
        k.load(b, bS)
        k.mma(c, a, b, c)
        k.sync()

    k.store(cS, c)
    k.storeGlobal(cPtr, cS, coord)
    return k.build()


def _flash_attn_fwd_2block(name: str, out_kind: str, numKvBlocks: int = 2) -> Kernel:
    """The three 2-block forward programs of Tyr/GPU/Kernels/MhaH100.lean share everything but their
    second output: none (`tkFlashAttnFwd2Block`, :14-68), LSE = ln(l) + m (`tkFlashAttnFwd2BlockLse`,
    :71-128) or L = -8 LSE, the ThunderKittens convention for D = 64 (`tkMhaH100Fwd2Block`, :130-190)."""
    k = KernelBuilder(name)
    q_ptr = k.gptr("BFloat16", "q_ptr")
    k_ptr = k.gptr("BFloat16", "k_ptr")
    v_ptr = k.gptr("BFloat16", "v_ptr")
    o_ptr = k.gptr("BFloat16", "o_ptr")
    vec_ptr = k.gptr("Float32", "lse_ptr" if out_kind == "lse" else "l_ptr") if out_kind != "none" else None
    k.kval("UInt64", "_seq_len")
    k.kval("UInt64", "_head_dim")
    tileSize = 64
    scale = 0.125

    coord = k.blockCoord2D()

    q = k.allocRT("BFloat16", tileSize, tileSize)
    kt = k.allocRT("BFloat16", tileSize, tileSize)
    v = k.allocRT("BFloat16", tileSize, tileSize, "Col")
    o = k.zeroRT("Float32", tileSize, tileSize)

    softmaxState = k.allocSoftmaxState("Float32", tileSize)

    qShared = k.allocST("BFloat16", tileSize, tileSize)
    kShared = k.allocST("BFloat16", tileSize, tileSize)
    vShared = k.allocST("BFloat16", tileSize, tileSize, "Col")
    oShared = k.allocST("BFloat16", tileSize, tileSize)
    vecShared = k.allocSV("Float32", tileSize) if out_kind != "none" else None

    k.loadGlobal(qShared, q_ptr, coord)
    k.sync()
    k.load(q, qShared)

    with k.krange(0, numKvBlocks) as kvIdx:
        s = k.zeroRT("Float32", tileSize, tileSize)
        p = k.allocRT("BFloat16", tileSize, tileSize)

        k.loadGlobal(kShared, k_ptr, coord.withRow(kvIdx.id))
        k.loadGlobal(vShared, v_ptr, coord.withRow(kvIdx.id))
        k.sync()
        k.load(kt, kShared)
        k.load(v, vShared)

        k.mmaT(s, q, kt, s)
        k.scalarMul(s, s, scale)
        k.onlineSoftmax(s, o, softmaxState)
        k.convert(p, s)
        k.mma(o, p, v, o)
        k.sync()

    k.finalizeSoftmax(o, softmaxState)
    if out_kind != "none":
        lse = k.computeLSE(softmaxState)
        if out_kind == "l":
            k.scalarMulVec(lse, lse, -8.0)

    oBf16 = k.allocRT("BFloat16", tileSize, tileSize)
    k.convert(oBf16, o)
    k.store(oShared, oBf16)
    k.storeGlobal(o_ptr, oShared, coord)

    if out_kind != "none":
        k.storeVec(vecShared, lse)
        k.storeVecGlobalRow(vec_ptr, vecShared, coord)
    return k.build()


def tkFlashAttnFwd2Block() -> Kernel:
    return _flash_attn_fwd_2block("tkFlashAttnFwd2Block", "none")


def tkFlashAttnFwd2BlockLse() -> Kernel:
    return _flash_attn_fwd_2block("tkFlashAttnFwd2BlockLse", "lse")


def tkMhaH100Fwd2Block() -> Kernel:
    return _flash_attn_fwd_2block("tkMhaH100Fwd2Block", "l")


def tkFlashAttnFwd12Block() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100.lean:347-398 -- the same program over 12 KV blocks (seq = 768)."""
    return _flash_attn_fwd_2block("tkFlashAttnFwd12Block", "none", 12)


def tkFlashAttnFwd12BlockLse() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100.lean:400-457."""
    return _flash_attn_fwd_2block("tkFlashAttnFwd12BlockLse", "lse", 12)


def tkMhaH100Fwd12Block() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100.lean:459-519."""
    return _flash_attn_fwd_2block("tkMhaH100Fwd12Block", "l", 12)


def tkMhaH100BwdPrep2Block() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100.lean:192-227 -- d[row] = sum_j dO[row, j] * O[row, j]."""
    k = KernelBuilder("tkMhaH100BwdPrep2Block")
    dO_ptr = k.gptr("BFloat16", "dO_ptr")
    o_ptr = k.gptr("BFloat16", "o_ptr")
    d_ptr = k.gptr("Float32", "d_ptr")
    k.kval("UInt64", "_seq_len")
    k.kval("UInt64", "_head_dim")
    tileSize = 64
    coord = k.blockCoord2D()

    dO = k.allocRT("BFloat16", tileSize, tileSize)
    o = k.allocRT("BFloat16", tileSize, tileSize)
    dOf = k.allocRT("Float32", tileSize, tileSize)
    of = k.allocRT("Float32", tileSize, tileSize)
    prod = k.allocRT("Float32", tileSize, tileSize)
    dVec = k.allocRV("Float32", tileSize)

    dOShared = k.allocST("BFloat16", tileSize, tileSize)
    oShared = k.allocST("BFloat16", tileSize, tileSize)
    dShared = k.allocSV("Float32", tileSize)

    k.loadGlobal(dOShared, dO_ptr, coord)
    k.loadGlobal(oShared, o_ptr, coord)
    k.sync()
    k.load(dO, dOShared)
    k.load(o, oShared)

    k.convert(dOf, dO)
    k.convert(of, o)
    k.mul(prod, dOf, of)
    k.rowSum(dVec, prod)

    k.storeVec(dShared, dVec)
    k.storeVecGlobalRow(d_ptr, dShared, coord)
    return k.build()


def tkMhaH100Bwd2BlockPartials(name: str = "tkMhaH100Bwd2BlockPartials", numKvBlocks: int = 2) -> Kernel:
    """Tyr/GPU/Kernels/MhaH100.lean:229-344 -- backward of one 64-row query tile over two KV blocks
    (non-causal): dQ final, dK / dV as one 64x64 partial per (kv tile, q tile) that the caller sums
    over q tiles (Examples/GPU/RunMhaH100.lean:131-138).  Scores are kept in K x Q orientation."""
    k = KernelBuilder(name)
    q_ptr = k.gptr("BFloat16", "q_ptr")
    k_ptr = k.gptr("BFloat16", "k_ptr")
    v_ptr = k.gptr("BFloat16", "v_ptr")
    dO_ptr = k.gptr("BFloat16", "dO_ptr")
    l_ptr = k.gptr("Float32", "l_ptr")
    d_ptr = k.gptr("Float32", "d_ptr")
    dQ_ptr = k.gptr("Float32", "dQ_ptr")
    dK_part_ptr = k.gptr("Float32", "dK_part_ptr")
    dV_part_ptr = k.gptr("Float32", "dV_part_ptr")
    k.kval("UInt64", "_seq_len")
    k.kval("UInt64", "_head_dim")
    tileSize = 64
    scale = 0.125
    invLScale = -0.125

    coord = k.blockCoord2D()

    q = k.allocRT("BFloat16", tileSize, tileSize)
    dO = k.allocRT("BFloat16", tileSize, tileSize)
    dQ = k.zeroRT("Float32", tileSize, tileSize)
    lTk = k.allocRV("Float32", tileSize)
    lse = k.allocRV("Float32", tileSize)
    dVec = k.allocRV("Float32", tileSize)

    rowShared = k.allocST("BFloat16", tileSize, tileSize)
    colShared = k.allocST("BFloat16", tileSize, tileSize, "Col")
    outShared = k.allocST("Float32", tileSize, tileSize)
    vecShared = k.allocSV("Float32", tileSize)

    k.loadGlobal(rowShared, q_ptr, coord)
    k.sync()
    k.load(q, rowShared)
    k.loadGlobal(rowShared, dO_ptr, coord)
    k.sync()
    k.load(dO, rowShared)

    k.loadVecGlobalRow(vecShared, l_ptr, coord)
    k.sync()
    k.loadVec(lTk, vecShared)
    k.loadVecGlobalRow(vecShared, d_ptr, coord)
    k.sync()
    k.loadVec(dVec, vecShared)
    k.scalarMulVec(lse, lTk, invLScale)

    with k.krange(0, numKvBlocks) as kvIdx:
        kk = k.allocRT("BFloat16", tileSize, tileSize)
        v = k.allocRT("BFloat16", tileSize, tileSize, "Col")
        sT = k.zeroRT("Float32", tileSize, tileSize)
        pT = k.allocRT("Float32", tileSize, tileSize)
        dPT = k.zeroRT("Float32", tileSize, tileSize)
        dST = k.allocRT("Float32", tileSize, tileSize)
        dKPart = k.zeroRT("Float32", tileSize, tileSize)
        dVPart = k.zeroRT("Float32", tileSize, tileSize)

        k.loadGlobal(rowShared, k_ptr, coord.withRow(kvIdx.id))
        k.loadGlobal(colShared, v_ptr, coord.withRow(kvIdx.id))
        k.sync()
        k.load(kk, rowShared)
        k.load(v, colShared)

        k.mmaT(sT, kk, q, sT)
        k.scalarMul(sT, sT, scale)
        k.subRow(sT, sT, lse)
        k.exp(pT, sT)

        vRow = k.allocRT("BFloat16", tileSize, tileSize)
        k.swapLayout(vRow, v)
        k.mmaT(dPT, vRow, dO, dPT)
        k.subRow(dPT, dPT, dVec)

        k.mul(dST, pT, dPT)
        dSTScaled = k.allocRT("Float32", tileSize, tileSize)
        k.scalarMul(dSTScaled, dST, scale)

        pTBf16 = k.allocRT("BFloat16", tileSize, tileSize)
        k.convert(pTBf16, pT)
        dSTBf16 = k.allocRT("BFloat16", tileSize, tileSize)
        k.convert(dSTBf16, dSTScaled)

        dOCol = k.allocRT("BFloat16", tileSize, tileSize, "Col")
        k.swapLayout(dOCol, dO)
        k.mma(dVPart, pTBf16, dOCol, dVPart)

        qCol = k.allocRT("BFloat16", tileSize, tileSize, "Col")
        k.swapLayout(qCol, q)
        k.mma(dKPart, dSTBf16, qCol, dKPart)

        dSRow = k.allocRT("BFloat16", tileSize, tileSize)
        k.transpose(dSRow, dSTBf16)
        kCol = k.allocRT("BFloat16", tileSize, tileSize, "Col")
        k.swapLayout(kCol, kk)
        k.mma(dQ, dSRow, kCol, dQ)

        dkvCoord = coord.withRow(kvIdx.id).withCol(coord.r)
        k.store(outShared, dKPart)
        k.sync()
        k.storeGlobal(dK_part_ptr, outShared, dkvCoord)
        k.store(outShared, dVPart)
        k.sync()
        k.storeGlobal(dV_part_ptr, outShared, dkvCoord)
        k.sync()

    k.store(outShared, dQ)
    k.sync()
    k.storeGlobal(dQ_ptr, outShared, coord)
    return k.build()


def tkMhaH100Bwd12BlockPartials() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100.lean:521-640 -- the backward program over 12 KV blocks (seq = 768)."""
    return tkMhaH100Bwd2BlockPartials("tkMhaH100Bwd12BlockPartials", 12)


def _mhaH100LcfFwd(name: str, headDim: int, kvTileRows: int, numKvTiles: int, banner: str, scale: float) -> Kernel:
    """Tyr/GPU/Kernels/MhaH100LCF.lean:29-82 -- one stationary 64 x D query tile, KV streamed in tiles of
    kvTileRows rows, online softmax across the stream."""
    k = KernelBuilder(name)
    q_ptr = k.gptr("BFloat16", "q_ptr")
    k_ptr = k.gptr("BFloat16", "k_ptr")
    v_ptr = k.gptr("BFloat16", "v_ptr")
    o_ptr = k.gptr("BFloat16", "o_ptr")
    k.kval("UInt64", "_seq_len")
    k.kval("UInt64", "_head_dim")
    k.comment(banner)
    k.comment("ThunderKittens lcf pipeline compressed into a typed single-query-tile shell")
    k.comment("The exact multi-worker CTA packing is still flattened to one logical query tile per kernel instance.")

    coord = k.blockCoord2D()

    qShared = k.allocST("BFloat16", 64, headDim)
    kShared = k.allocST("BFloat16", kvTileRows, headDim)
    vShared = k.allocST("BFloat16", kvTileRows, headDim, "Col")
    oShared = k.allocST("BFloat16", 64, headDim)

    q = k.allocRT("BFloat16", 64, headDim)
    kt = k.allocRT("BFloat16", kvTileRows, headDim)
    v = k.allocRT("BFloat16", kvTileRows, headDim, "Col")
    o = k.zeroRT("Float32", 64, headDim)
    softmaxState = k.allocSoftmaxState("Float32", 64)

    k.loadGlobal(qShared, q_ptr, coord)
    k.sync()
    k.load(q, qShared)

    with k.krange(0, numKvTiles) as kvIdx:
        kvCoord = coord.withRow(kvIdx.id)
        scores = k.zeroRT("Float32", 64, kvTileRows)
        probs = k.allocRT("BFloat16", 64, kvTileRows)

        k.loadGlobal(kShared, k_ptr, kvCoord)
        k.loadGlobal(vShared, v_ptr, kvCoord)
        k.sync()
        k.load(kt, kShared)
        k.load(v, vShared)

        k.mmaT(scores, q, kt, scores)
        k.scalarMul(scores, scores, scale)
        k.onlineSoftmax(scores, o, softmaxState)
        k.convert(probs, scores)
        k.mma(o, probs, v, o)
        k.sync()

    k.finalizeSoftmax(o, softmaxState)
    oBf16 = k.allocRT("BFloat16", 64, headDim)
    k.convert(oBf16, o)
    k.store(oShared, oBf16)
    k.storeGlobal(o_ptr, oShared, coord)
    return k.build()


def tkMhaH100LCFFwd64() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100LCF.lean:84-107 -- D = 64, KV tiles of 192 rows, 3072 / 192 = 16 of them."""
    return _mhaH100LcfFwd("tkMhaH100LCFFwd64", 64, 192, 16,
                          "=== ThunderKittens mha_h100_lcf forward (D=64, KV tile 192) ===", 0.125)


def tkMhaH100LCFFwd128() -> Kernel:
    """Tyr/GPU/Kernels/MhaH100LCF.lean:109-132 -- D = 128, KV tiles of 128 rows, 3072 / 128 = 24 of them."""
    return _mhaH100LcfFwd("tkMhaH100LCFFwd128", 128, 128, 24,
                          "=== ThunderKittens mha_h100_lcf forward (D=128, KV tile 128) ===", 0.08838834764)


def tkH100Bf16GemmFwd() -> Kernel:
    """Tyr/GPU/Kernels/Bf16Gemm.lean:19-73 over GemmCommon.lean:22-69 -- C tile 128 x 256 from A [128, 64] and
    B [256, 64] (B is N x K) slices over 4 K blocks, f32 accumulate, bf16 out."""
    k = KernelBuilder("tkH100Bf16GemmFwd")
    aPtr = k.gptr("BFloat16", "aPtr")
    bPtr = k.gptr("BFloat16", "bPtr")
    cPtr = k.gptr("BFloat16", "cPtr")
    k.kval("UInt64", "m")
    k.kval("UInt64", "n")
    k.kval("UInt64", "k")
    accum, coord = _tiledAccumulator(
        k, "=== H100 BF16 GEMM ===",
        "ThunderKittens bf16_h100 producer/consumer tile, expressed as a single CTA-local tiled mainloop",
        aPtr, bPtr, "BFloat16", 128, 64, 256, 4)
    # storeConvertedTile (GemmCommon.lean:58-69)
    out = k.allocRT("BFloat16", 128, 256)
    outShared = k.allocST("BFloat16", 128, 256)
    k.convert(out, accum)
    k.store(outShared, out)
    k.storeGlobal(cPtr, outShared, coord)
    return k.build()


def _tiledAccumulator(k: KernelBuilder, banner, sourceNote, aPtr, bPtr, inDtype, tileM, tileK, tileN, kBlocks):
    """Tyr/GPU/Kernels/GemmCommon.lean:22-56 -- A tile [tileM, tileK], B tile [tileN, tileK] (B is N x K),
    f32 accumulator over kBlocks slices."""
    k.comment(banner)
    k.comment(sourceNote)
    k.comment(f"Tile shape: A {tileM}x{tileK}, B {tileN}x{tileK}, C {tileM}x{tileN}")
    coord = k.blockCoord2D()
    a = k.allocRT(inDtype, tileM, tileK)
    b = k.allocRT(inDtype, tileN, tileK)
    accum = k.zeroRT("Float32", tileM, tileN)
    aShared = k.allocST(inDtype, tileM, tileK)
    bShared = k.allocST(inDtype, tileN, tileK)
    with k.krange(0, kBlocks) as kBlk:
        aCoord = coord.withCol(kBlk.id)
        bCoord = coord.withRow(coord.c).withCol(kBlk.id)
        k.loadGlobal(aShared, aPtr, aCoord)
        k.loadGlobal(bShared, bPtr, bCoord)
        k.sync()
        k.load(a, aShared)
        k.load(b, bShared)
        k.mmaT(accum, a, b, accum)
        k.sync()
    return accum, coord


def _h100Fp8Accumulator(k, banner, aPtr, bPtr):
    """Tyr/GPU/Kernels/PrecisionGemm.lean:26-49 -- 64 x 256 output tile, k in 4 slices of 128."""
    return _tiledAccumulator(k, banner, "ThunderKittens fp8_h100 tile family", aPtr, bPtr, "FP8E4M3", 64, 128, 256, 4)


def gemmFp8E4M3Fwd() -> Kernel:
    """Tyr/GPU/Kernels/PrecisionGemm.lean:178-189 with GemmCommon.storeConvertedTile (GemmCommon.lean:58-69):
    E4M3 x E4M3 -> f32 -> bf16, C tile 64 x 256, K = 512."""
    k = KernelBuilder("gemmFp8E4M3Fwd")
    aPtr = k.gptr("FP8E4M3", "aPtr")
    bPtr = k.gptr("FP8E4M3", "bPtr")
    cPtr = k.gptr("BFloat16", "cPtr")
    k.kval("UInt64", "m")
    k.kval("UInt64", "n")
    k.kval("UInt64", "k")
    accum, coord = _h100Fp8Accumulator(k, "=== H100 FP8 GEMM compatibility epilogue (E4M3 -> BF16) ===", aPtr, bPtr)
    out = k.allocRT("BFloat16", 64, 256)
    outShared = k.allocST("BFloat16", 64, 256)
    k.convert(out, accum)
    k.store(outShared, out)
    k.storeGlobal(cPtr, outShared, coord)
    return k.build()


def tkH100Fp8ScaledGemmFwd() -> Kernel:
    """Tyr/GPU/Kernels/PrecisionGemm.lean:97-115 -- the same mainloop, then per-row scales of A and
    per-column scales of B on the f32 accumulator (GemmCommon.lean:71-84, 123-133), f32 out."""
    k = KernelBuilder("tkH100Fp8ScaledGemmFwd")
    aPtr = k.gptr("FP8E4M3", "aPtr")
    bPtr = k.gptr("FP8E4M3", "bPtr")
    scaleAPtr = k.gptr("Float32", "scaleAPtr")
    scaleBPtr = k.gptr("Float32", "scaleBPtr")
    cPtr = k.gptr("Float32", "cPtr")
    k.kval("UInt64", "m")
    k.kval("UInt64", "n")
    k.kval("UInt64", "k")
    accum, coord = _h100Fp8Accumulator(k, "=== H100 FP8 GEMM with row/column scales ===", aPtr, bPtr)
    scaleRowShared = k.allocSV("Float32", 64)
    scaleColShared = k.allocSV("Float32", 256)
    scaleRow = k.allocRV("Float32", 64)
    scaleCol = k.allocRV("Float32", 256)
    k.loadVecGlobalRow(scaleRowShared, scaleAPtr, coord)
    k.loadVecGlobalCol(scaleColShared, scaleBPtr, coord)
    k.loadVec(scaleRow, scaleRowShared)
    k.loadVec(scaleCol, scaleColShared)
    scaled = k.allocRT("Float32", 64, 256)
    k.mulCol(scaled, accum, scaleRow)
    k.mulRow(scaled, scaled, scaleCol)
    outShared = k.allocST("Float32", 64, 256)
    k.store(outShared, scaled)
    k.storeGlobal(cPtr, outShared, coord)
    return k.build()


def _causal_demo_attn_fwd(name: str, banner: str, with_lse: bool, explicit_softmax: bool) -> Kernel:
    """The reference's three demonstration forwards with `makeCausal` share one shape: 64 x 64 tiles, four KV blocks, no
    score scale, the per-tile causal mask with fill -1e10, and a score tile that is allocated once outside the loop and
    *accumulated into* by every `mmaT s q k s` (it is never cleared: the scores of block j start from the probabilities of
    block j-1, and from the tile's initial contents -- zeros in this lowering -- for block 0).
      flashAttnFwdNew      Tyr/GPU/Kernels/FlashAttn.lean:26-95      onlineSoftmax / finalizeSoftmax macros
      flashAttnFwdWithLse  Tyr/GPU/Kernels/FlashAttnBwd.lean:25-103  the same, plus LSE = ln(l) + m per row
      flashAttnFwd         Tyr/GPU/Kernels/Examples.lean:93-144      running row max / row sum without rescaling O"""
    k = KernelBuilder(name)
    q_ptr = k.gptr("BFloat16", "q_ptr")
    k_ptr = k.gptr("BFloat16", "k_ptr")
    v_ptr = k.gptr("BFloat16", "v_ptr")
    o_ptr = k.gptr("BFloat16", "o_ptr")
    l_ptr = k.gptr("Float32", "l_ptr") if with_lse else None
    k.kval("UInt64", "_seq_len")
    k.kval("UInt64", "_head_dim")
    if banner:
        k.comment(banner)
    coord = k.blockCoord2D()
    q = k.allocRT("BFloat16", 64, 64)
    kt = k.allocRT("BFloat16", 64, 64)
    v = k.allocRT("BFloat16", 64, 64, "Col")
    s_ = k.allocRT("Float32", 64, 64)
    p = k.allocRT("BFloat16", 64, 64)
    o = k.zeroRT("Float32", 64, 64)
    if explicit_softmax:
        rowMax = k.negInftyRV("Float32", 64)
        rowSum = k.allocRV("Float32", 64)
    else:
        state = k.allocSoftmaxState("Float32", 64)
    qS = k.allocST("BFloat16", 64, 64)
    kS = k.allocST("BFloat16", 64, 64)
    vS = k.allocST("BFloat16", 64, 64, "Col")
    oS = k.allocST("BFloat16", 64, 64)
    lS = k.allocSV("Float32", 64) if with_lse else None
    k.loadGlobal(qS, q_ptr, coord)
    k.sync()
    k.load(q, qS)
    with k.krange(0, 4) as kv:
        k.loadGlobal(kS, k_ptr, coord.withRow(kv.id))
        k.loadGlobal(vS, v_ptr, coord.withRow(kv.id))
        k.sync()
        k.load(kt, kS)
        k.load(v, vS)
        k.mmaT(s_, q, kt, s_)
        k.makeCausal(s_, s_, -1e10)
        if explicit_softmax:
            k.rowMaxAccum(rowMax, s_, rowMax)
            k.subCol(s_, s_, rowMax)
            k.exp(s_, s_)
            k.rowSumAccum(rowSum, s_, rowSum)
        else:
            k.onlineSoftmax(s_, o, state)
        k.convert(p, s_)
        k.mma(o, p, v, o)
        k.sync()
    if explicit_softmax:
        k.divCol(o, o, rowSum)
    else:
        k.finalizeSoftmax(o, state)
        if with_lse:
            lse = k.computeLSE(state)
    oBf16 = k.allocRT("BFloat16", 64, 64)
    k.convert(oBf16, o)
    k.store(oS, oBf16)
    k.storeGlobal(o_ptr, oS, coord)
    if with_lse:
        k.storeVec(lS, lse)
        k.storeVecGlobalRow(l_ptr, lS, coord)
    return k.build()


def flashAttnFwdNew() -> Kernel:
    return _causal_demo_attn_fwd("flashAttnFwdNew", "=== FlashAttention Forward ===", False, False)


def flashAttnFwdWithLse() -> Kernel:
    return _causal_demo_attn_fwd("flashAttnFwdWithLse", "=== FlashAttention Forward (with LSE for backward) ===", True, False)


def flashAttnFwd() -> Kernel:
    return _causal_demo_attn_fwd("flashAttnFwd", "", False, True)


def simpleGemmNew() -> Kernel:
    """Tyr/GPU/Kernels/FlashAttn.lean:98-131 -- the test GEMM of that file: the program of `simpleGemm` under its own name."""
    k = simpleGemm()
    k.name = "simpleGemmNew"
    return k


def tkH100Fp8E4M3GemmFwd() -> Kernel:
    """Tyr/GPU/Kernels/PrecisionGemm.lean:73-89 with GemmCommon.storeConvertedTile (GemmCommon.lean:58-69): the canonical
    H100 FP8 surface, E4M3 x E4M3 -> f32 -> E4M3 on 64 x 256 output tiles, K = 512."""
    k = KernelBuilder("tkH100Fp8E4M3GemmFwd")
    aPtr = k.gptr("FP8E4M3", "aPtr")
    bPtr = k.gptr("FP8E4M3", "bPtr")
    cPtr = k.gptr("FP8E4M3", "cPtr")
    k.kval("UInt64", "m")
    k.kval("UInt64", "n")
    k.kval("UInt64", "k")
    accum, coord = _h100Fp8Accumulator(k, "=== H100 FP8 GEMM (E4M3 -> E4M3 epilogue) ===", aPtr, bPtr)
    out = k.allocRT("FP8E4M3", 64, 256)
    outShared = k.allocST("FP8E4M3", 64, 256)
    k.convert(out, accum)
    k.store(outShared, out)
    k.storeGlobal(cPtr, outShared, coord)
    return k.build()


def tkB200Fp8E4M3Gemm1CtaFwd() -> Kernel:
    """Tyr/GPU/Kernels/PrecisionGemm.lean:117-133 (accumulator :52-69): the Blackwell one-CTA surface, E4M3 x E4M3 -> f32 ->
    bf16 on 128 x 256 output tiles, K = 512.  Nothing in the program is specific to that device; on gfx950 it is run by a
    group of four waves with B read from LDS, like the H100 bf16 surface."""
    k = KernelBuilder("tkB200Fp8E4M3Gemm1CtaFwd")
    aPtr = k.gptr("FP8E4M3", "aPtr")
    bPtr = k.gptr("FP8E4M3", "bPtr")
    dPtr = k.gptr("BFloat16", "dPtr")
    k.kval("UInt64", "m")
    k.kval("UInt64", "n")
    k.kval("UInt64", "k")
    accum, coord = _tiledAccumulator(
        k, "=== B200 FP8 GEMM (1 CTA) ===",
        "ThunderKittens fp8_b200_gemm_1cta reduced to a typed 128x256 Blackwell-sized CTA mainloop",
        aPtr, bPtr, "FP8E4M3", 128, 128, 256, 4)
    out = k.allocRT("BFloat16", 128, 256)
    outShared = k.allocST("BFloat16", 128, 256)
    k.convert(out, accum)
    k.store(outShared, out)
    k.storeGlobal(dPtr, outShared, coord)
    return k.build()


# kernel name -> the reference definition it restates
CITES = {
    "copy64x64": "Tyr/GPU/Kernels/Copy.lean:16-26 (runner Examples/GPU/RunCopy.lean:28)",
    "rotaryFwd": "Tyr/GPU/Kernels/Rotary.lean:13-62 (runner Examples/GPU/RunRotary.lean:63)",
    "tkFusedLayerNormResidual1024": "Tyr/GPU/Kernels/FusedLayerNorm.lean:28-126 (runner Examples/GPU/RunLayerNorm.lean:67)",
    "simpleGemm": "Tyr/GPU/Kernels/Examples.lean:23-65",
    "gemmFp8E4M3Fwd": "Tyr/GPU/Kernels/PrecisionGemm.lean:178-189 over GemmCommon.lean:22-69",
    "tkH100Fp8ScaledGemmFwd": "Tyr/GPU/Kernels/PrecisionGemm.lean:97-115 over GemmCommon.lean:22-133",
    "tkFlashAttnFwd2Block": "Tyr/GPU/Kernels/MhaH100.lean:14-68 (runner Examples/GPU/RunFlashAttn.lean:80)",
    "tkFlashAttnFwd2BlockLse": "Tyr/GPU/Kernels/MhaH100.lean:71-128 (runner Examples/GPU/RunFlashAttn.lean:81)",
    "tkMhaH100Fwd2Block": "Tyr/GPU/Kernels/MhaH100.lean:130-190 (runner Examples/GPU/RunMhaH100.lean:112)",
    "tkMhaH100BwdPrep2Block": "Tyr/GPU/Kernels/MhaH100.lean:192-227 (runner Examples/GPU/RunMhaH100.lean:119)",
    "tkMhaH100Bwd2BlockPartials": "Tyr/GPU/Kernels/MhaH100.lean:229-344 (runner Examples/GPU/RunMhaH100.lean:126)",
    "tkFlashAttnFwd12Block": "Tyr/GPU/Kernels/MhaH100.lean:347-398",
    "tkFlashAttnFwd12BlockLse": "Tyr/GPU/Kernels/MhaH100.lean:400-457 (runner Examples/GPU/RunMhaH100Seq768.lean:102)",
    "tkMhaH100Fwd12Block": "Tyr/GPU/Kernels/MhaH100.lean:459-519 (runner Examples/GPU/RunMhaH100Seq768.lean:108)",
    "tkMhaH100Bwd12BlockPartials": "Tyr/GPU/Kernels/MhaH100.lean:521-640 (runner Examples/GPU/RunMhaH100Seq768.lean:119)",
    "tkMhaH100LCFFwd64": "Tyr/GPU/Kernels/MhaH100LCF.lean:84-107 (run by a group of 2 waves, K and V read from LDS by the products)",
    "tkMhaH100LCFFwd128": "Tyr/GPU/Kernels/MhaH100LCF.lean:109-132 (run by a group of 2 waves, K and V read from LDS by the products)",
    "tkH100Bf16GemmFwd": "Tyr/GPU/Kernels/Bf16Gemm.lean:64-73 over GemmCommon.lean:22-69 (run by a group of 4 waves, B read from LDS by the products)",
    "flashAttnFwdNew": "Tyr/GPU/Kernels/FlashAttn.lean:26-95",
    "flashAttnFwdWithLse": "Tyr/GPU/Kernels/FlashAttnBwd.lean:25-103",
    "flashAttnFwd": "Tyr/GPU/Kernels/Examples.lean:93-144",
    "simpleGemmNew": "Tyr/GPU/Kernels/FlashAttn.lean:98-131",
    "tkH100Fp8E4M3GemmFwd": "Tyr/GPU/Kernels/PrecisionGemm.lean:73-89 over GemmCommon.lean:22-69",
    "tkB200Fp8E4M3Gemm1CtaFwd": "Tyr/GPU/Kernels/PrecisionGemm.lean:117-133 over GemmCommon.lean:22-69 (run by a group of 4 waves, B read from LDS by the products)",
}
ALL = (copy64x64, rotaryFwd, tkFusedLayerNormResidual1024, simpleGemm, gemmFp8E4M3Fwd, tkH100Fp8ScaledGemmFwd,
       tkFlashAttnFwd2Block, tkFlashAttnFwd2BlockLse,
       tkMhaH100Fwd2Block, tkMhaH100BwdPrep2Block, tkMhaH100Bwd2BlockPartials,
       tkFlashAttnFwd12Block, tkFlashAttnFwd12BlockLse, tkMhaH100Fwd12Block, tkMhaH100Bwd12BlockPartials,
       tkMhaH100LCFFwd64, tkMhaH100LCFFwd128, tkH100Bf16GemmFwd,
       flashAttnFwdNew, flashAttnFwdWithLse, flashAttnFwd, simpleGemmNew, tkH100Fp8E4M3GemmFwd, tkB200Fp8E4M3Gemm1CtaFwd)
