// Implicit-GEMM convolution on the fp32 matrix cores (v_mfma_f32_32x32x2f32), stride 1, N = 1:
// conv3d 3x3x3 pad 1, conv2d 3x3 pad 1, conv 1x1, and the 2x2 stride-2 transposed conv (as a 1x1
// conv with 4F output channels whose epilogue scatters to (2y+a, 2x+b)).  Bias / folded
// BatchNorm / activation / residual are applied in the epilogue.
//
// Replaces k_conv3d_direct3 (runtime/fortis_fft.cu:148-201: scalar FMA from shared memory, 32
// accumulators per thread) and the cuDNN calls of runtime/fortis_rt.c:108-156.
//
// GEMM view: rows = output channels (MFMA A operand = weights), columns = output positions (B operand
// = input patches), k = (input channel, tap).  One MFMA step multiplies two input channels (the two
// lane halves) at one tap.
// Positions are linearised inside one z-plane with pitch P = W + 1: m = y*P + x.  On the virtual
// zero-padded plane of the same pitch (the right pad of a row is the left pad of the next), tap
// (kh, kw) of position m is element m + kh*P + kw: a lane-independent offset.  A workgroup therefore
// stages, per input channel and per kd, ONE contiguous run of MT + 2P + 2 virtual elements into LDS
// (zero-filled outside the image), and every B operand is a single ds_read at lane base + constant.
// Weights are re-packed once at plan time in exactly the order the kernel consumes them, so their
// staging is a straight 16-byte copy.  Both are double buffered through registers.
// On wide 2-D images that run is mostly halo (two whole rows for one tile's worth of positions), so 3 x 3
// convs on images at least 64 wide use a second tiling (TILE2D): a workgroup's positions are MT / 32 rows of
// 32 columns, staged with a one-pixel border at a fixed pitch of 34, tap (kh, kw) = element + kh*34 + kw.
#include <type_traits>
#include "stencil_dev.h"      // StMagic / st_divmod: exact division by a launch constant

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float cm_v4f __attribute__((ext_vector_type(4)));   // native vector: conditional copies stay in registers

#define CM_THREADS 256
// Input channels per staged chunk.  A chunk's multiply phase has to outlast the latency of the next
// chunk's global loads: with 9 or 27 taps 4 channels do, a single tap takes 16.  (8 channels at 9 taps
// gain 10% on 32 x 32 images and lose 30% on 256 x 256 ones, whose halo then no longer fits the larger tile.)
static constexpr int cm_cc(int T) { return T >= 27 ? 2 : T >= 9 ? 4 : 16; }
#ifndef CM_STORE_NUM
#define CM_STORE_NUM 6    // eighths of a chunk's products in front of the move of the next chunk into LDS (TSRGAN step, 8: 1.871 ms, 7: 1.873, 6: 1.858, 5: 1.876, 4: 1.872)
#endif
#ifndef CM_DEFER
#define CM_DEFER 4         // products of a chunk kept behind the step's barrier (TSRGAN step, 0: 1.850 ms, 2: 1.845, 4: 1.839, 6: 1.849, 8: 1.888)
#endif
#define CM_NXMAX 16   // staging rounds of the input run, at most (the kernel is built for 8 and for 16)

struct ConvMShape {
    int C, D, H, W, F;         // F = output channels of the GEMM (4x the real ones in transposed mode)
    int P, plane, tiles, nchunks, R;
    int tiles_x;               // TILE2D: tiles along x
    int mode;                  // 0: convolution, 1: 2x2 stride-2 transposed conv scatter
    int ksplit;                // channel chunks are split over blockIdx.z; > 1: raw partial sums go to `part`
    int cbase, cextra;         // slice k takes cbase chunks, the first cextra slices one more (larger slices first: they are dispatched first)
    float* part;               // [ksplit][output elements]
    int sk_per, sk_items;      // streamed split: (tile, chunk) items per workgroup and in all (per group of output channels)
    int sk_tile0;              // streamed split: its first tile (the tiles before it are computed whole by a launch of their own)
    int ups;                   // 1: the input tensor is (D/2, H/2, W/2) and is read through a nearest x2 upsample
    long osize;                // output elements
    StMagic mP, mR, mKR;       // exact division by P, R and KD * R (the staging map would otherwise spend its time dividing)
    StMagic mT, mTX, mNC, mPer; // ... by tiles, tiles_x, nchunks and sk_per (a scalar division costs some forty instructions at the head of every workgroup)
};

// FT output channels per workgroup: 64 (waves 2 x 2 over channels x positions) or 32 (4 waves over positions).
// Workgroup barrier that orders LDS traffic only: global loads already issued stay in flight across it.
__device__ __forceinline__ void cm_lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

#define CM_TP 34       // TILE2D: pitch of a staged row (32 columns + border)
// KG > 1: the workgroup's waves also divide the input channels of every chunk among KG groups; each group
// accumulates the same output tile over its channels and the groups' sums are added through LDS at the end, in
// group order.  This is how a launch with few output tiles (deep, small images) still puts four waves on every
// CU without partial sums in HBM and a second kernel: the tile shrinks to 32 x 32 and KG = 4.  KG = 2 (64 x 32
// tiles: two rows of 32 columns, each wave pair halves the channels) is the same trade for launches of one to five
// 64 x 64 tiles per CU: more, smaller workgroups keep the matrix pipes fed while others stage.
// SK (streamed split, volumes with fewer tiles than the chip needs): the launch's work is the list of (tile, chunk)
// items, tile-major; every workgroup takes the same count of consecutive items, whatever tile boundaries fall
// inside its run, and leaves one partial sum per tile it touched, in its accumulators' own register order
// (part[slot][tile][register][thread], slot = the workgroup's rank among those that share the tile).
// conv_sk_reduce_kernel adds a tile's slots in order and applies the epilogue.  Equal runs are what a split into
// whole slices cannot give: 297 tiles in 3 slices are 891 workgroups, four on some CUs and three on others.
// POOL: 0, 1 (the kernel also writes the 2 x 2 max pool of its tiles) or 2 (instead of its own output the kernel writes a
// following 1 x 1 convolution to at most four channels, computed from the finished tile in LDS: a thin head costs no launch).
template <int KD, int KS, int MT, int FT, int NX, bool TILE2D, int KG = 1, int POOL = 0, bool SK = false>
__global__ __launch_bounds__(CM_THREADS) __attribute__((amdgpu_waves_per_eu(SK ? 2 : KD == 3 && MT == 128 && FT == 64 && NX <= 8 ? 4 : 1)))
void conv_mfma_kernel(const float* __restrict__ x, const float* __restrict__ wp,
                                                               float* __restrict__ y, ConvMShape s, ConvEpi e)
{
    constexpr int T = KD * KS * KS;
    constexpr int CC = cm_cc(T) * KG, NCP = CC / 2;  // NX: staging rounds of the input run (8 or 16)
    constexpr int NCPW = NCP / KG;                               // channel pairs of a chunk per channel group
    constexpr int WCH = NCP * T * 2 * FT;                        // floats of packed weights per chunk
    constexpr int NW = (WCH / 4 + CM_THREADS - 1) / CM_THREADS;  // float4 per thread
    constexpr int FW = FT / 32;                                  // waves along the channels
    constexpr int NMT = MT / 32 / (4 / (FW * KG));               // m-tiles per wave
    static_assert(NMT >= 1, "tile too small for the wave layout");
    static_assert(KG == 1 || NMT == 1, "channel groups: one m-tile per wave");
    constexpr int PADK = KS / 2;
    constexpr int TH = MT / 32, R2 = (TH + 2) * CM_TP;           // TILE2D: rows per tile, staged elements per channel
    static_assert(!TILE2D || (KD == 1 && KS == 3), "the 2-D tiling is for 3 x 3 convs");
    // XDUMP: a chunk's stores into LDS are unconditional -- an input element that is padding sends its (unused) value to
    // a spare slot behind the buffer's staged elements instead of being masked off, and the weights' buffer is padded
    // to whole rounds of the workgroup's 16-byte stores (WCHP; the padding receives copies of the chunk's first
    // weights and is never read).  One select per element and tile, where a mask costs a save, a branch and a restore
    // of the lane mask per element and chunk; and a steady-state step without branches is one block of code whose
    // loads and stores the scheduler can place between the matrix instructions (step_full).  Not in the form that runs
    // four workgroups per CU (its registers have none to spare for the addresses, its LDS none for the padding), nor
    // in the streamed one with 16 staging rounds.
    constexpr bool XDUMP = SK ? NX <= 8 : !(KD == 3 && MT == 128 && FT == 64 && NX <= 8);
    constexpr int WCHP = XDUMP ? NW * CM_THREADS * 4 : WCH;      // floats of LDS per weight buffer
    extern __shared__ float4 smem4[];
    float* sW = (float*)smem4;                                    // [2][WCHP]
    float* sX = sW + 2 * WCHP;                                    // [2][CC * KD * R rounded up to a wave's 64 lanes]
    const int RR = TILE2D ? R2 : KS == 1 ? MT : s.R;              // staged elements per channel and kd (s.R, a constant where it can be)
    const int XCH = CC * KD * RR;
    const int XCHP = (XCH + 64) / 64 * 64;                        // at least one spare slot behind the staged elements (see XDUMP)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // volumes: neighbouring tiles and planes on one XCD (input fetched once instead of 2-3 times; on images the
    // banded order measured 2 % slower)
    const int wgx = KD == 3 ? (int)fortis_xcd_band(blockIdx.x, gridDim.x) : (int)blockIdx.x;
    const int fg = blockIdx.y;
    static_assert(!SK || (KG == 1 && !POOL && !TILE2D), "the streamed split is for the plain volume kernel");
    int it = 0, itend = 0;                                        // SK: the workgroup's run of items
    if constexpr (SK) {
        it = wgx * s.sk_per;
        itend = it + s.sk_per < s.sk_items ? it + s.sk_per : s.sk_items;
    }
    for (;;) {                                                    // SK: once per tile of the run; otherwise once
    int bx = wgx, ch0, ch1;
    if constexpr (SK) {
        if (it >= itend) break;
        unsigned tq, cq;
        st_divmod((unsigned)it, s.mNC, tq, cq);
        bx = (int)tq + s.sk_tile0;
        ch0 = (int)cq;
        ch1 = ch0 + (itend - it) < s.nchunks ? ch0 + (itend - it) : s.nchunks;
    } else {
        const int kz = blockIdx.z;
        ch0 = kz * s.cbase + (kz < s.cextra ? kz : s.cextra);
        ch1 = ch0 + s.cbase + (kz < s.cextra ? 1 : 0);
    }
    unsigned zq = 0, tileq = (unsigned)bx, tyq = 0, txq = 0;
    if constexpr (KD != 1) st_divmod((unsigned)bx, s.mT, zq, tileq);          // images have one plane (the launcher sees to it)
    if constexpr (TILE2D) st_divmod(tileq, s.mTX, tyq, txq);
    const int z = (int)zq, tile = (int)tileq;
    const int m0 = tile * MT;
    const int tyi = (int)tyq, y0 = tyi * TH, x0 = (int)txq * 32;               // TILE2D: tile origin
    const long HW = (long)s.H * s.W, chan = (long)s.D * HW;
    // source geometry: the tensor itself, or the half-resolution tensor a fused nearest upsample reads
    const int sh = s.ups ? 1 : 0;
    const long srcW = s.W >> sh, sHW = (long)(s.H >> sh) * srcW, schan = (long)(s.D >> sh) * sHW;

    // Two register sets: while LDS holds chunk k, set (k+1)&1 carries chunk k+1 (loaded one step ago) and
    // set k&1 receives chunk k+2, so a chunk's global loads have two multiply phases to arrive in.
    struct Regs { cm_v4f rw[NW]; float rx[NX]; };
    Regs rg[2];
    auto load_weights = [&](Regs& r, int ch) {
        const cm_v4f* wsrc = (const cm_v4f*)(wp + ((long)fg * s.nchunks + ch) * WCH);
#pragma unroll
        for (int i = 0; i < NW; i++) {
            const int f4 = tid + i * CM_THREADS;
            r.rw[i] = wsrc[f4 < WCH / 4 ? f4 : 0];
        }
    };
    // the first chunk's weights need nothing of the staging map below: they are on their way while it is worked out
    load_weights(rg[0], ch0);
    // So are the epilogue's per-channel scale and shift for this workgroup's FT channels, which wait in LDS from the
    // first barrier on: fetched in the epilogue they cost every launch a round trip to memory after its last matrix
    // instruction.  (Not in the form that fills the CU's LDS with four workgroups, nor in the streamed one, whose
    // epilogue is the reduce kernel's.)
    constexpr bool EPILDS = !SK && !(KD == 3 && MT == 128 && FT == 64 && NX <= 8);
    __shared__ float sEpi[EPILDS ? 2 * FT : 1];
    float epi_sc = 1.f, epi_sf = 0.f;
    if constexpr (EPILDS) {
        if (tid < FT && s.ksplit == 1) {
            const int f = fg * FT + tid, fc = f < s.F ? f : 0, fo = s.mode ? fc >> 2 : fc;
            if (e.scale) epi_sc = e.scale[fo];
            if (e.shift) epi_sf = e.shift[fo];
        }
    }

    // per-thread staging map of the input run (same for every chunk): byte offset inside a chunk's channel
    // group, (c * schan + offset in the channel) * 4.  Padding elements load from offset 0 (goff) and carry
    // the mark 0xffffffff in gchk, which the store compares with the chunk's limit.
    unsigned goff[NX], gchk[NX];
    bool inb[NX];                // the element lies inside the tensor (not padding, not past the staged run)
    unsigned xslot[XDUMP ? NX : 1];
#pragma unroll
    for (int i = 0; i < NX; i++) {
        // straight-line: an element past the staged run or outside the tensor works its numbers out like any other
        // (nothing is read with them) and is switched off at the end
        const int el = tid + i * CM_THREADS;
        unsigned c, r, off;
        bool in = el < XCH;
        if constexpr (KD == 1 && KS == 1) {
            // a 1 x 1 conv stages MT consecutive positions of each channel: no borders, no row structure
            c = (unsigned)el / MT; r = (unsigned)el % MT;
            in = in && m0 + (int)r < s.plane;
            off = (unsigned)(c * schan + m0 + r) * 4u;
        } else {
            unsigned rem, kd, yp, xp;
            int zz, yy, xx;
            if (TILE2D) {
                c = (unsigned)el / R2; r = (unsigned)el % R2;    // compile-time divisors
                zz = z; yy = y0 + (int)(r / CM_TP) - 1; xx = x0 + (int)(r % CM_TP) - 1;
            } else {
                st_divmod((unsigned)el, s.mKR, c, rem);
                st_divmod(rem, s.mR, kd, r);
                st_divmod((unsigned)(m0 + r), s.mP, yp, xp);
                zz = z + (int)kd - (KD / 2); yy = (int)yp - PADK; xx = (int)xp - PADK;
            }
            in = in & ((unsigned)zz < (unsigned)s.D) & ((unsigned)yy < (unsigned)s.H) & ((unsigned)xx < (unsigned)s.W);
            off = (unsigned)(c * schan + (zz >> sh) * sHW + (long)(yy >> sh) * srcW + (xx >> sh)) * 4u;
        }
        goff[i] = in ? off : 0u;
        gchk[i] = in ? off : 0xffffffffu;
        inb[i] = in;
        if constexpr (XDUMP) xslot[i] = in ? (unsigned)el : (unsigned)XCH;
    }

    // byte offsets at or beyond chunk_lim belong to channels past the last one (only in a partial last chunk)
    auto chunk_lim = [&](int ch) {
        const int cleft = s.C - ch * CC;
        return (unsigned)((cleft < CC ? cleft : CC) * schan) * 4u;
    };
    auto load_input = [&](Regs& r, int ch) {
        // uniform base + 32-bit byte offset per lane: no address arithmetic here.  Padding elements read
        // offset 0 (a valid address); they are replaced by zero only when stored, so nothing waits here.
        const char* xsrc = (const char*)(x + (long)ch * CC * schan);
        if ((ch + 1) * CC > s.C) {
            // partial last chunk: channels past the last one read offset 0 too.  It is the last chunk this tile loads,
            // so the offsets are clamped in place (one load site; a second one with clamped copies cost every chunk a
            // move per offset where the two join)
            unsigned lim = chunk_lim(ch);
            asm volatile("" : "+s"(lim));            // opaque here: the clamps below cannot be hoisted out of the branch
#pragma unroll
            for (int i = 0; i < NX; i++) goff[i] = goff[i] < lim ? goff[i] : 0u;
        }
#pragma unroll
        for (int i = 0; i < NX; i++) r.rx[i] = *(const float*)(xsrc + goff[i]);
    };
    auto load_chunk = [&](Regs& r, int ch) { load_weights(r, ch); load_input(r, ch); };
    // An element that is padding is padding in every chunk: its LDS slots are zeroed once per tile (zero_padding) and
    // a chunk's store skips it under the lane mask `inb` (kept in scalar registers: no vector instruction per element,
    // where a select of the value against zero cost two).  Only a partial last chunk still selects: its channels past
    // the last one store zeros.
    auto store_chunk = [&](const Regs& r, int buf, int ch) {
        cm_v4f* wdst = (cm_v4f*)(sW + buf * WCHP);
#pragma unroll
        for (int i = 0; i < NW; i++) {
            const int f4 = tid + i * CM_THREADS;
            if (XDUMP || f4 < WCH / 4) wdst[f4] = r.rw[i];
        }
        float* xdst = sX + buf * XCHP + tid;
        if ((ch + 1) * CC <= s.C) {
            if constexpr (XDUMP) {
                float* xb = sX + buf * XCHP;
#pragma unroll
                for (int i = 0; i < NX; i++) xb[xslot[i]] = r.rx[i];
            } else {
#pragma unroll
                for (int i = 0; i < NX; i++)
                    if (inb[i]) xdst[i * CM_THREADS] = r.rx[i];
            }
        } else {
            const unsigned lim = chunk_lim(ch);
#pragma unroll
            for (int i = 0; i < NX; i++)
                if (inb[i]) xdst[i * CM_THREADS] = gchk[i] < lim ? r.rx[i] : 0.f;
        }
    };
    auto zero_padding = [&]() {
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < NX; i++)
                if (!inb[i] && tid + i * CM_THREADS < XCHP) sX[b * XCHP + tid + i * CM_THREADS] = 0.f;
    };

    const int kgi = wave % KG, wtile = wave / KG;                 // channel group; the wave's tile among the workgroup's
    const int ft = wtile % FW, mt0 = (wtile / FW) * NMT;
    const int wbase = (lane >> 5) * FT + ft * 32 + (lane & 31) + kgi * NCPW * T * 2 * FT;
    // lane's element for tap (0, 0) of its first m-tile; an m-tile is 32 consecutive positions of the run, or
    // (TILE2D) one row of the tile
    const int xbase = (lane >> 5) * KD * RR + mt0 * (TILE2D ? CM_TP : 32) + (lane & 31) + 2 * kgi * NCPW * KD * RR;
    v16f acc[NMT];
#pragma unroll
    for (int j = 0; j < NMT; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0.f;

    // products q0 <= q < q1 of the chunk's NCPW * T (channel pair, tap) products, in order
    auto multiply_part = [&](int buf, const int q0, const int q1) __attribute__((always_inline)) {
        const float* w = sW + buf * WCHP + wbase;
        const float* xs = sX + buf * XCHP + xbase;
#pragma unroll
        for (int cp = 0; cp < NCPW; cp++)
#pragma unroll
            for (int kd = 0; kd < KD; kd++)
#pragma unroll
                for (int kh = 0; kh < KS; kh++)
#pragma unroll
                    for (int kw = 0; kw < KS; kw++) {
                        const int tap = (kd * KS + kh) * KS + kw;
                        if (cp * T + tap < q0 || cp * T + tap >= q1) continue;
                        const float a = w[(cp * T + tap) * 2 * FT];
                        const int xoff = (2 * cp * KD + kd) * RR + kh * (TILE2D ? CM_TP : s.P) + kw;
#pragma unroll
                        for (int j = 0; j < NMT; j++)
                            acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, xs[j * (TILE2D ? CM_TP : 32) + xoff], acc[j], 0, 0, 0);
                    }
    };
    auto multiply = [&](int buf) __attribute__((always_inline)) { multiply_part(buf, 0, NCPW * T); };
    // The chunk's last ND products wait behind the step's barrier with their operands already in registers: they are what
    // the matrix pipe has to do while the workgroup's waves meet and the next chunk's first operands come out of LDS.
    // (Not in the form whose 128 registers have none to spare.)
    constexpr int ND = (XDUMP || SK) && NCPW * T > 2 * CM_DEFER ? CM_DEFER : 0;
    float dfa[ND > 0 ? ND : 1], dfx[ND > 0 ? ND : 1][NMT];
    auto preread_last = [&](int buf) __attribute__((always_inline)) {
        const float* w = sW + buf * WCHP + wbase;
        const float* xs = sX + buf * XCHP + xbase;
#pragma unroll
        for (int d = 0; d < ND; d++) {
            const int q = NCPW * T - ND + d, cp = q / T, tap = q % T;
            const int kd = tap / (KS * KS), kh = (tap / KS) % KS, kw = tap % KS;
            dfa[d] = w[(cp * T + tap) * 2 * FT];
            const int xoff = (2 * cp * KD + kd) * RR + kh * (TILE2D ? CM_TP : s.P) + kw;
#pragma unroll
            for (int j = 0; j < NMT; j++) dfx[d][j] = xs[j * (TILE2D ? CM_TP : 32) + xoff];
        }
    };
    auto multiply_last = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int d = 0; d < ND; d++)
#pragma unroll
            for (int j = 0; j < NMT; j++)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(dfa[d], dfx[d][j], acc[j], 0, 0, 0);
    };
    // the product behind which a step moves the next chunk into LDS (the rest of the chunk's products then run
    // beside those stores instead of in front of them)
    constexpr int QS = NCPW * T * CM_STORE_NUM / 8;
    // One step of the pipeline on chunk ch (LDS buffer buf): fetch chunk ch + 2 into `far`, multiply, move
    // chunk ch + 1 from `near` into the other LDS buffer.  The steady-state form is unconditional: the
    // compiler's wait insertion counts loads behind a branch as possibly absent and would then wait for
    // the newest loads where only the oldest are needed.
    // (only where a wave is alone or nearly alone on its SIMD: the forms whose four waves divide the input channels,
    // at one or two workgroups per CU.  With three or four waves per SIMD the other waves fill those gaps anyway and
    // the block order with the multiply phase at raised priority measured 2-3 % faster.)
    constexpr bool INTERLEAVE = XDUMP && KG == 4;
    auto step_full = [&](int ch, int buf, Regs& far, const Regs& near) {
        if constexpr (INTERLEAVE) {
            // Neither chunk ch + 1 nor ch + 2 is a partial one here (the loop below sees to it), so the step has no
            // branch: the loads of chunk ch + 2 and the stores of chunk ch + 1 (into the LDS buffer nobody reads during
            // this step) are spread between the matrix instructions.  Issued in a block in front of and behind them,
            // a workgroup's 25 KB of loads hold its four waves at the CU's one address unit for 400-500 cycles and the
            // stores for 300-400, beside 1152 cycles of matrix work per chunk: a wave alone on its SIMD multiplied
            // half the time.
            load_weights(far, ch + 2);
            {
                const char* xsrc = (const char*)(x + (long)(ch + 2) * CC * schan);
#pragma unroll
                for (int i = 0; i < NX; i++) far.rx[i] = *(const float*)(xsrc + goff[i]);
            }
            multiply(buf);
            {
                cm_v4f* wdst = (cm_v4f*)(sW + (buf ^ 1) * WCHP);
#pragma unroll
                for (int i = 0; i < NW; i++) wdst[tid + i * CM_THREADS] = near.rw[i];
                float* xb = sX + (buf ^ 1) * XCHP;
#pragma unroll
                for (int i = 0; i < NX; i++) xb[xslot[i]] = near.rx[i];
            }
            constexpr int NMF = NCPW * T * NMT, NMOVE = NW + NX;          // matrix instructions; loads = stores
            // loads behind the first matrix instructions, stores behind the later ones, evenly
#pragma unroll
            for (int m = 0; m < NMF; m++) {
                __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);        // LDS reads (operands a little ahead)
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        // one matrix instruction
                constexpr int H = NMF / 2;
                if (m < H) {
                    const int a = m * NMOVE / H, b = (m + 1) * NMOVE / H;
                    if (b - a >= 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    if (b - a >= 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    if (b - a >= 3) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                } else {
                    const int a = (m - H) * NMOVE / (NMF - H), b = (m - H + 1) * NMOVE / (NMF - H);
                    if (b - a >= 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                    if (b - a >= 2) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                    if (b - a >= 3) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                }
            }
            cm_lds_barrier();
        } else {
        load_chunk(far, ch + 2);
        __builtin_amdgcn_sched_barrier(0);     // nothing of the store below (it waits for `near`) moves above the multiplies
        // the multiply phase outranks the other resident waves' staging at the issue port (UNet 0.266 -> 0.262 ms)
        __builtin_amdgcn_s_setprio(2);
        multiply_part(buf, 0, QS);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        store_chunk(near, buf ^ 1, ch + 1);
        if constexpr (QS < NCPW * T) {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(2);
            multiply_part(buf, QS, NCPW * T - ND);
            __builtin_amdgcn_s_setprio(0);
        }
        if constexpr (ND > 0) preread_last(buf);
        cm_lds_barrier();
        if constexpr (ND > 0) {
            __builtin_amdgcn_sched_barrier(0);
            multiply_last();
        }
        }
    };
    auto step_tail = [&](int ch, int buf, Regs& far, const Regs& near) {
        if (ch + 2 < ch1) load_chunk(far, ch + 2);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(2);
        multiply(buf);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        if (ch + 1 < ch1) store_chunk(near, buf ^ 1, ch + 1);
        cm_lds_barrier();
    };
    load_input(rg[0], ch0);
    zero_padding();
    if constexpr (EPILDS) {
        if (tid < FT) { sEpi[tid] = epi_sc; sEpi[FT + tid] = epi_sf; }
    }
    store_chunk(rg[0], 0, ch0);
    cm_lds_barrier();
    load_chunk(rg[1], ch0 + 1 < ch1 ? ch0 + 1 : ch0);     // unconditional for the same reason (a lone chunk is fetched twice)
    int ch = ch0;
    // the unconditional steps stop short of a partial last chunk (fewer than CC channels left), which only
    // the tail steps load and store
    const int chfull = INTERLEAVE && s.nchunks * CC > s.C && ch1 == s.nchunks ? ch1 - 1 : ch1;
    for (; ch + 3 < chfull; ch += 2) {
        step_full(ch, 0, rg[0], rg[1]);
        step_full(ch + 1, 1, rg[1], rg[0]);
    }
    for (; ch < ch1; ch += 2) {
        step_tail(ch, 0, rg[0], rg[1]);
        if (ch + 1 < ch1) step_tail(ch + 1, 1, rg[1], rg[0]);
    }

    // epilogue: a lane holds one position and 16 output channels per m-tile
    const long ospatial = s.mode ? 4 * chan : chan;
    // Registers r0 .. r0 + N - 1 of m-tile j at once.  Every step of the epilogue runs over all of them before the next
    // begins (a step's loads, from addresses clamped into the tensors, leave together and are waited for once; the
    // null checks of the epilogue's pointers are taken once, not per element).  Per element the operations and their
    // order are those of the reference's fused epilogue: scale, shift, activation, residual.
    auto finish_regs = [&](const int j, const int r0, auto nc, float* v) __attribute__((always_inline)) {
        constexpr int N = decltype(nc)::value;
        unsigned yy, xx;
        bool inside;
        if (TILE2D) {
            yy = (unsigned)(y0 + mt0 + j); xx = (unsigned)(x0 + (lane & 31));
            inside = (int)yy < s.H;
        } else {
            const int m = m0 + (mt0 + j) * 32 + (lane & 31);
            inside = m < s.plane;
            st_divmod((unsigned)(inside ? m : 0), s.mP, yy, xx);
        }
        inside = inside && (int)xx < s.W;
        if (!inside) { yy = 0; xx = 0; }
        const int fb = fg * FT + ft * 32 + 4 * (lane >> 5);
        const unsigned opos = (unsigned)(((long)z * s.H + yy) * s.W + xx);
        int fo[N];
        unsigned off[N];             // element offsets: the launcher keeps every tensor below 2^31 elements
        bool ok[N];
#pragma unroll
        for (int q = 0; q < N; q++) {
            const int r = r0 + q, f = fb + 8 * (r >> 2) + (r & 3);
            ok[q] = inside && f < s.F;
            const int fc = f < s.F ? f : 0;
            if (s.mode) {
                fo[q] = fc >> 2;
                off[q] = (unsigned)(fo[q] * ospatial) + (2 * yy + ((fc >> 1) & 1)) * (2 * s.W) + 2 * xx + (fc & 1);
            } else {
                fo[q] = fc;
                off[q] = (unsigned)(fc * ospatial) + opos;
            }
        }
        if (s.ksplit > 1) {
            float* part = s.part + blockIdx.z * s.osize;
#pragma unroll
            for (int q = 0; q < N; q++) if (ok[q]) part[off[q]] = v[q];
            return;
        }
        float t[N];
        if (e.scale) {
#pragma unroll
            for (int q = 0; q < N; q++) {
                const int r = r0 + q;
                t[q] = EPILDS ? sEpi[ft * 32 + 4 * (lane >> 5) + 8 * (r >> 2) + (r & 3)] : e.scale[fo[q]];
            }
#pragma unroll
            for (int q = 0; q < N; q++) v[q] = v[q] * t[q];
        }
        if (e.shift) {
#pragma unroll
            for (int q = 0; q < N; q++) {
                const int r = r0 + q;
                t[q] = EPILDS ? sEpi[FT + ft * 32 + 4 * (lane >> 5) + 8 * (r >> 2) + (r & 3)] : e.shift[fo[q]];
            }
#pragma unroll
            for (int q = 0; q < N; q++) v[q] = v[q] + t[q];
        }
        if (e.act == FORTIS_ACT_RELU) {
#pragma unroll
            for (int q = 0; q < N; q++) v[q] = v[q] > 0.f ? v[q] : 0.f;
        } else if (e.act == FORTIS_ACT_LEAKY) {
#pragma unroll
            for (int q = 0; q < N; q++) v[q] = v[q] > 0.f ? v[q] : e.alpha * v[q];
        }
        if (e.res) {
#pragma unroll
            for (int q = 0; q < N; q++) t[q] = e.res[off[q]];
#pragma unroll
            for (int q = 0; q < N; q++) v[q] = v[q] + t[q];
        }
#pragma unroll
        for (int q = 0; q < N; q++) {
            if (!ok[q]) continue;
            if constexpr (POOL != 2) y[off[q]] = v[q];
            if constexpr (POOL != 0) {
                // the finished tile also goes to LDS as [channel][row][32 columns] for the 2 x 2 max pool below
                // (behind the channel groups' sums, which other waves may still be reading)
                const int r = r0 + q, f = fb + 8 * (r >> 2) + (r & 3);
                ((float*)smem4)[(KG > 1 ? 4 * 16 * 64 : 0) + ((f - fg * FT) * TH + (mt0 + j)) * 32 + (lane & 31)] = v[q];
            }
        }
    };
    // 2 x 2 stride-2 max pool of the finished tile (H and W even, tiles start on even rows and columns: a 2 x 2
    // block lies inside the image or outside it as a whole); staging has ended, LDS is free
    auto pool_tile = [&]() __attribute__((always_inline)) {
        if constexpr (POOL == 2) {
            // head: out[o][pos] = head_b[o] + sum over this conv's channels of head_w[o][c] * tile[c][pos], channels in order
            cm_lds_barrier();
            const float* pt = (const float*)smem4 + (KG > 1 ? 4 * 16 * 64 : 0);
            const int nh = e.head_n;
            for (int idx = tid; idx < nh * MT; idx += CM_THREADS) {
                const int pos = idx % MT, o = idx / MT, row = pos >> 5, col = pos & 31;
                const int yy = y0 + row, xx = x0 + col;
                if (yy >= s.H || xx >= s.W) continue;
                float a = e.head_b ? e.head_b[o] : 0.f;
                const float* hw = e.head_w + o * s.F;
                for (int c = 0; c < s.F; c++) a = fmaf(hw[c], pt[(c * TH + row) * 32 + col], a);
                e.head_y[((long)o * s.H + yy) * s.W + xx] = a;
            }
        }
        if constexpr (POOL == 1) {
            cm_lds_barrier();
            const float* pt = (const float*)smem4 + (KG > 1 ? 4 * 16 * 64 : 0);
            const int Ho = s.H >> 1, Wo = s.W >> 1;
            for (int idx = tid; idx < FT * (TH / 2) * 16; idx += CM_THREADS) {
                const int pc = idx & 15, pr = (idx >> 4) % (TH / 2), fl = idx / (16 * (TH / 2));
                const int f = fg * FT + fl, yo = (y0 >> 1) + pr, xo = (x0 >> 1) + pc;
                if (f >= s.F || yo >= Ho || xo >= Wo) continue;
                const float* q = pt + (fl * TH + 2 * pr) * 32 + 2 * pc;
                const float m0 = q[0] > q[1] ? q[0] : q[1], m1 = q[32] > q[33] ? q[32] : q[33];
                e.pool[((long)f * Ho + yo) * Wo + xo] = m0 > m1 ? m0 : m1;
            }
        }
    };
    static_assert(POOL != 1 || (TILE2D && (MT / 32) % 2 == 0), "the in-kernel pool needs the 32-column tiling and an even tile height");
    static_assert(POOL != 2 || TILE2D, "the in-kernel head needs the 32-column tiling");
    if constexpr (SK) {
        // the accumulators as they are: slot = this workgroup's rank among those whose runs share the tile
        const int tl = bx - s.sk_tile0;
        unsigned w0q, rr;
        st_divmod((unsigned)(tl * s.nchunks), s.mPer, w0q, rr);
        const int slot = wgx - (int)w0q;
        float* pd = s.part + (((long)slot * gridDim.y + fg) * (s.D * s.tiles - s.sk_tile0) + tl) * (NMT * 16 * CM_THREADS) + tid;
        // (a register at a time, 256 consecutive bytes per wave, as device-scope stores: written through L2 as they are
        // issued instead of lingering there dirty; TSRGAN step 1.897 -> 1.873 ms against 16-byte plain stores.  Letting
        // the workgroup that brings a tile's last sum finish the tile, counted in through a device-scope atomic, instead
        // of the second kernel measured 2.02 ms: the waits for the stores and the atomic, and the finishing at the
        // kernel's tail, cost more than the 9 us launch they replace)
#pragma unroll
        for (int j = 0; j < NMT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                __hip_atomic_store(pd + (j * 16 + r) * CM_THREADS, acc[j][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        it += ch1 - ch0;
        continue;
    } else if constexpr (KG == 1) {
        // registers finished at a time: all 16 of an m-tile, or 4 in the form that keeps four workgroups on a CU
        // (its 128 registers have no room for 16 offsets and 16 loaded values beside the accumulators)
        constexpr int EN = (KD == 3 && MT == 128 && FT == 64 && NX <= 8) ? 4 : 16;
#pragma unroll
        for (int j = 0; j < NMT; j++)
#pragma unroll
            for (int r0 = 0; r0 < 16; r0 += EN) {
                float v[EN];
#pragma unroll
                for (int q = 0; q < EN; q++) v[q] = acc[j][r0 + q];
                finish_regs(j, r0, std::integral_constant<int, EN>(), v);
            }
        if constexpr (POOL) pool_tile();
    } else {
        // the loop above ended on a barrier: the staging buffers are free.  red[tile][group][register][lane]
        float* red = (float*)smem4 + wtile * (KG * 16 * 64);
#pragma unroll
        for (int r = 0; r < 16; r++) red[(kgi * 16 + r) * 64 + lane] = acc[0][r];
        cm_lds_barrier();
        // group g finishes registers g * 16 / KG ...: the groups' sums are added in group order
        float v[16 / KG];
#pragma unroll
        for (int q = 0; q < 16 / KG; q++) {
            const int r = kgi * (16 / KG) + q;
            v[q] = red[r * 64 + lane];
#pragma unroll
            for (int g = 1; g < KG; g++) v[q] += red[(g * 16 + r) * 64 + lane];
        }
        finish_regs(0, kgi * (16 / KG), std::integral_constant<int, 16 / KG>(), v);
        if constexpr (POOL) pool_tile();
    }
    break;
    }
}

// The streamed split's finish: a tile's partial sums are added in slot order, i.e. in the order of the input
// channels, then the epilogue.  Threads as in conv_mfma_kernel (the same registers of the same lanes); rq names a group
// of four accumulator registers.  part[slot][channel group][tile][register][thread]; ntl tiles and nfg channel
// groups are streamed, a tile's items meet nseg runs.
template <int MT, int FT>
__device__ __forceinline__ void conv_sk_finish_quad(float* __restrict__ y, const ConvMShape& s, const ConvEpi& e, const int tl, const int fg,
                                                    const int ntl, const int nfg, const int nseg, const int rq, const int tid)
{
    constexpr int FW = FT / 32, NMT = MT / 32 / (4 / FW), NQ = NMT * 4;
    const int lane = tid & 63, wave = tid >> 6;
    const long slot = (long)ntl * nfg * (NQ * 4 * CM_THREADS);
    const float* p = s.part + (((long)fg * ntl + tl) * NQ + rq) * (4 * CM_THREADS) + tid;
    // a thread's loads all leave before the first is needed: the first four slots (a tile always has two) and the
    // residual values; the sums are then added in slot order
    auto ld4 = [&](const long off) __attribute__((always_inline)) {
        cm_v4f v;
#pragma unroll
        for (int q = 0; q < 4; q++) v[q] = p[off + q * CM_THREADS];
        return v;
    };
    const cm_v4f a0 = ld4(0), a1 = ld4(nseg > 1 ? slot : 0);
    const cm_v4f a2 = ld4(nseg > 2 ? 2 * slot : 0), a3 = ld4(nseg > 3 ? 3 * slot : 0);
    unsigned zq, tileq;
    st_divmod((unsigned)(tl + s.sk_tile0), s.mT, zq, tileq);
    const int z = (int)zq, tile = (int)tileq;
    const int ft = wave % FW, mt0 = (wave / FW) * NMT;
    const long ospatial = (long)s.D * s.H * s.W;
    const int m = tile * MT + (mt0 + rq / 4) * 32 + (lane & 31);
    unsigned yy, xx;
    st_divmod((unsigned)m, s.mP, yy, xx);
    const bool inside = m < s.plane && (int)xx < s.W;
    const long opos = inside ? ((long)z * s.H + yy) * s.W + xx : 0;
    const int f0 = fg * FT + ft * 32 + 8 * (rq & 3) + 4 * (lane >> 5);             // registers 4 * (rq & 3) ... + 3 of the m-tile
    float res[4], sc[4], sf[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int fc = f0 + q < s.F ? f0 + q : 0;
        res[q] = e.res ? e.res[fc * ospatial + opos] : 0.f;
        sc[q] = e.scale ? e.scale[fc] : 0.f;
        sf[q] = e.shift ? e.shift[fc] : 0.f;
    }
    cm_v4f acc = a0;
    if (nseg > 1) acc += a1;
    if (nseg > 2) acc += a2;
    if (nseg > 3) acc += a3;
    for (int k = 4; k < nseg; k++) acc += ld4(k * slot);
    if (!inside) return;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int f = f0 + q;
        if (f >= s.F) continue;
        float v = acc[q];
        if (e.scale) v = v * sc[q];
        if (e.shift) v = v + sf[q];
        if (e.act == FORTIS_ACT_RELU) v = v > 0.f ? v : 0.f;
        else if (e.act == FORTIS_ACT_LEAKY) v = v > 0.f ? v : e.alpha * v;
        if (e.res) v = v + res[q];
        y[f * ospatial + opos] = v;
    }
}
// Runs of the streamed split that meet tile tl.
__device__ __forceinline__ int conv_sk_nseg(const ConvMShape& s, const int tl)
{
    const int first = tl * s.nchunks;
    unsigned w0q, w1q, rr;
    st_divmod((unsigned)first, s.mPer, w0q, rr);
    st_divmod((unsigned)(first + s.nchunks - 1), s.mPer, w1q, rr);
    return (int)(w1q - w0q) + 1;
}

// Second kernel of the streamed split, for launches with more tiles than there are counters: a workgroup per tile and
// group of four accumulator registers (a tile alone would be too few workgroups for a kernel that only moves memory).
#define CM_RQB 2      // register quads per workgroup of the reduce kernel
template <int MT, int FT>
__global__ __launch_bounds__(CM_THREADS) void conv_sk_reduce_kernel(float* __restrict__ y, ConvMShape s, ConvEpi e)
{
    const int tl = blockIdx.x, fg = blockIdx.y, tid = threadIdx.x;
    const int nseg = conv_sk_nseg(s, tl);
    // a workgroup takes CM_RQB register quads of its tile, one after the other in the code and together in flight
#pragma unroll
    for (int u = 0; u < CM_RQB; u++)
        conv_sk_finish_quad<MT, FT>(y, s, e, tl, fg, (int)gridDim.x, (int)gridDim.y, nseg, (int)blockIdx.z * CM_RQB + u, tid);
}

// Sums the partial results of a channel-split launch in split order (deterministic) and applies the
// epilogue.  ospatial = elements per output channel.  V = 4: a thread takes four consecutive elements of one
// channel (ospatial a multiple of 4, all pointers 16-byte aligned).
template <int V>
__global__ void conv_split_reduce_kernel(const float* __restrict__ part, float* __restrict__ y, long osize, long ospatial,
                                         int ksplit, ConvEpi e)
{
    const long idx = ((long)blockIdx.x * blockDim.x + threadIdx.x) * V;
    if (idx >= osize) return;
    float v[V];
    if constexpr (V == 4) {
        float4 a = *(const float4*)(part + idx);
        for (int k = 1; k < ksplit; k++) {
            const float4 q = *(const float4*)(part + k * osize + idx);
            a.x += q.x; a.y += q.y; a.z += q.z; a.w += q.w;
        }
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    } else {
        v[0] = part[idx];
        for (int k = 1; k < ksplit; k++) v[0] += part[k * osize + idx];
    }
    const long fo = idx / ospatial;
    const float sc = e.scale ? e.scale[fo] : 1.f, sf = e.shift ? e.shift[fo] : 0.f;
    float r[V];
    if constexpr (V == 4) {
        const float4 q = e.res ? *(const float4*)(e.res + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
        r[0] = q.x; r[1] = q.y; r[2] = q.z; r[3] = q.w;
    } else {
        r[0] = e.res ? e.res[idx] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < V; i++) {
        float t = v[i];
        if (e.scale) t = t * sc;
        if (e.shift) t = t + sf;
        if (e.act == FORTIS_ACT_RELU) t = t > 0.f ? t : 0.f;
        else if (e.act == FORTIS_ACT_LEAKY) t = t > 0.f ? t : e.alpha * t;
        if (e.res) t = t + r[i];
        v[i] = t;
    }
    if constexpr (V == 4) *(float4*)(y + idx) = make_float4(v[0], v[1], v[2], v[3]);
    else y[idx] = v[0];
}

static void launch_split_reduce(const float* part, float* y, long osize, long ospatial, int ksplit, const ConvEpi& e, hipStream_t st)
{
    const bool v4 = ospatial % 4 == 0 && (((uintptr_t)part | (uintptr_t)y | (uintptr_t)e.res) & 15) == 0;
    if (v4)
        hipLaunchKernelGGL(conv_split_reduce_kernel<4>, dim3((unsigned)cdiv(osize / 4, 256)), dim3(256), 0, st, part, y, osize,
                           ospatial, ksplit, e);
    else
        hipLaunchKernelGGL(conv_split_reduce_kernel<1>, dim3((unsigned)cdiv(osize, 256)), dim3(256), 0, st, part, y, osize, ospatial,
                           ksplit, e);
}

// The same for a 2-D conv whose output also goes through a 2 x 2 stride-2 max pool: a thread owns one pooled
// position, i.e. a 2 x 2 block of the output, writes its four values and their maximum.
__global__ void conv_split_reduce_pool_kernel(const float* __restrict__ part, float* __restrict__ y, float* __restrict__ pool,
                                              int F, int H, int W, long osize, int ksplit, ConvEpi e)
{
    const int Ho = H / 2, Wo = W / 2;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)F * Ho * Wo) return;
    const int xo = (int)(idx % Wo), yo = (int)((idx / Wo) % Ho);
    const long f = idx / ((long)Wo * Ho);
    const float sc = e.scale ? e.scale[f] : 1.f, sf = e.shift ? e.shift[f] : 0.f;
    float m = -INFINITY;
#pragma unroll
    for (int a = 0; a < 2; a++) {
        const long row = (f * H + 2 * yo + a) * W + 2 * xo;        // even: the pair is 8-byte aligned
        float2 v = *(const float2*)(part + row);
        for (int k = 1; k < ksplit; k++) { const float2 q = *(const float2*)(part + k * osize + row); v.x += q.x; v.y += q.y; }
        float o[2] = { v.x, v.y };
#pragma unroll
        for (int b = 0; b < 2; b++) {
            float t = o[b];
            if (e.scale) t = t * sc;
            if (e.shift) t = t + sf;
            if (e.act == FORTIS_ACT_RELU) t = t > 0.f ? t : 0.f;
            else if (e.act == FORTIS_ACT_LEAKY) t = t > 0.f ? t : e.alpha * t;
            if (e.res) t = t + e.res[row + b];
            o[b] = t;
            m = t > m ? t : m;
        }
        *(float2*)(y + row) = make_float2(o[0], o[1]);
    }
    pool[idx] = m;
}

// ---- host side ---------------------------------------------------------------------------------------
static inline long conv_ft(long Fg) { return Fg <= 32 ? 32 : 64; }
static int conv_cus()
{
    static int n = 0;
    if (!n) {
        hipDeviceProp_t prop;
        n = hipGetDeviceProperties(&prop, 0) == hipSuccess ? prop.multiProcessorCount : 256;
    }
    return n;
}

// A caller-provided workspace replaces the two buffers this file otherwise grows with fortis_dev_malloc (the packed
// weights of fortis_conv_mfma_pack_dev first, the partial sums of channel-split launches behind them) until it is
// taken away again with (null, 0).  A request that does not fit returns null, which the launchers turn into -1
// before anything is launched, and is remembered for fortis_conv_workspace_overflowed().
static char* g_ws = nullptr;
static size_t g_ws_bytes = 0, g_ws_pack = 0, g_ws_wanted = 0;
void fortis_conv_workspace(void* base, size_t bytes) { g_ws = (char*)base; g_ws_bytes = bytes; g_ws_pack = 0; g_ws_wanted = 0; }
size_t fortis_conv_workspace_overflowed() { return g_ws_wanted; }
static float* ws_take(size_t offset, size_t need)
{
    if (offset + need > g_ws_bytes) { g_ws_wanted = offset + need; return nullptr; }
    return (float*)(g_ws + offset);
}

// Partial sums of channel-split launches: one buffer for every shape (launches on the library's stream run
// one after the other).  It grows on the first, eager run of a plan; replays and captured runs find it in
// place.  An outgrown buffer stays allocated: a graph captured earlier may still name it.
static float* g_split = nullptr;   // the partial sums' buffer and the packed weights' one, with their sizes
static size_t g_split_cap = 0;
static float* g_pack = nullptr;
static size_t g_pack_cap = 0;
// The raw allocator was swapped (a test's hook): buffers of the old allocator are forgotten, not freed.
void fortis_conv_forget_buffers() { g_split = g_pack = nullptr; g_split_cap = g_pack_cap = 0; }
// Grows the partial sums' buffer ahead of time (a caller about to capture a graph; tests of the allocation
// path): 0, or -1 when the device has no memory for it.
extern "C" int fortis_conv_scratch_reserve(long bytes) { return bytes >= 0 && fortis_conv_split_scratch((size_t)bytes) ? 0 : -1; }

float* fortis_conv_split_scratch(size_t need)
{
    if (g_ws) return ws_take(g_ws_pack, need);
    float*& scratch = g_split;
    size_t& cap = g_split_cap;
    if (need > cap || !scratch) {
        float* p = nullptr;
        if (fortis_dev_malloc((void**)&p, need, "conv partial sums") != 0) return nullptr;
        scratch = p;
        cap = need;
    }
    return scratch;
}

int fortis_launch_conv_split_reduce(const float* part, float* y, long osize, long ospatial, int ksplit, const ConvEpi& e,
                                    hipStream_t st)
{
    launch_split_reduce(part, y, osize, ospatial, ksplit, e, st);
    HIP_OK(hipGetLastError());
    return 0;
}

// Channel groups inside a workgroup (the kernel's KG) for a conv on images with at least 32 input channels, by the
// number of 64 x 64 output tiles the launch would have: fewer than one per CU -> 4 (32 x 32 tiles whose four waves
// divide the input channels; the launch would otherwise be split over the input channels into partial sums and a
// reduce kernel); fewer than five per CU -> 2 (64 x 32 tiles, two waves per half of the channels:
// twice to four times the workgroups of the plain form, which at one or two workgroups per CU leaves the matrix
// pipes idle while a workgroup stages); 1 otherwise.  Fg: output channels of the GEMM (4 F for the transposed conv).
// Weights are packed for the answer, so packing and launching ask with the same arguments.
int fortis_conv_mfma_kgroups(long C, long D, long H, long Wd, long Fg, int KD, int KS, bool pooled)
{
    static const int off = getenv("FORTIS_CONV_KGROUPS") != nullptr && atoi(getenv("FORTIS_CONV_KGROUPS")) == 0;
    if (off || KD != 1 || D != 1 || C < 32) return 1;
    if (KS == 3 && !(Wd >= 32 && cdiv(Wd, 32) * 32 * 4 <= 5L * Wd)) return 1;     // 3 x 3: the 32-column tiling only
    if (KS != 1 && KS != 3) return 1;
    const long pos = KS == 3 ? H * (Wd + 1) : H * Wd, tiles = cdiv(pos, 64) * cdiv(Fg, 64);
    // (a 3 x 3 conv with a 2 x 2 max pool behind it takes the 64 x 32 form, which pools its own two-row tiles, rather
    // than the 32 x 32 one and a pool launch)
    static const int pool_kg2 = getenv("FORTIS_CONV_POOL_KG2") ? atoi(getenv("FORTIS_CONV_POOL_KG2")) : 1;
    if (tiles < conv_cus()) return pooled && pool_kg2 && KS == 3 && !(H & 1) && !(Wd & 1) && tiles * 2 >= conv_cus() ? 2 : 4;
    if (tiles < 5L * conv_cus()) return 2;
    return 1;
}

// Whether the launcher writes a following thin 1 x 1 convolution (nh output channels) from this conv's finished tiles:
// the 3 x 3 form with 64 x 32 tiles whose workgroup holds all of the conv's channels.
bool fortis_conv_mfma_head_ok(long C, long H, long Wd, long F, int KD, int KS, int nh)
{
    return KD == 1 && KS == 3 && F <= 32 && nh >= 1 && nh <= 4 && fortis_conv_mfma_kgroups(C, 1, H, Wd, F, 1, 3) == 2;
}

// Packs conv weights W[F][C][T] (T taps, row-major) into the kernel's order
//   [F/FT][ceil(C/CC)][channel pair CC/2][tap T][half 2][FT channels], zero padded; CC = cm_cc(T) * kg
//   channels per chunk; FT = 32 when the GEMM has at most 32 output channels or kg > 1, else 64 (the launcher
//   applies the same rules; kg = fortis_conv_mfma_kgroups of the shape).
// Transposed 2x2 conv: W is [C][F][2][2]; GEMM channel f' = f*4 + a*2 + b.
float* fortis_conv_mfma_pack(const float* W, long F, long C, int T, int transposed, long* nfloats, int kg)
{
    const long Fg = transposed ? 4 * F : F;
    const long FT = kg > 1 ? 32 : conv_ft(Fg);
    const long CC = cm_cc(T) * kg, NCP = CC / 2;
    const long nfg = cdiv(Fg, FT), nch = cdiv(C, CC);
    const long wch = NCP * T * 2 * FT;
    const long n = nfg * nch * wch;
    float* h = (float*)calloc(n, sizeof(float));
    for (long fgi = 0; fgi < nfg; fgi++)
        for (long ch = 0; ch < nch; ch++)
            for (int cp = 0; cp < NCP; cp++)
                for (int t = 0; t < T; t++)
                    for (int hh = 0; hh < 2; hh++)
                        for (int fl = 0; fl < FT; fl++) {
                            const long f = fgi * FT + fl, c = ch * CC + cp * 2 + hh;
                            if (f >= Fg || c >= C) continue;
                            const float v = transposed ? W[(c * F + (f >> 2)) * 4 + (f & 3)] : W[(f * C + c) * T + t];
                            h[((fgi * nch + ch) * NCP + cp) * T * 2 * FT + ((long)t * 2 + hh) * FT + fl] = v;
                        }
    float* d = nullptr;
    if (fortis_dev_malloc((void**)&d, n * sizeof(float), "packed conv weights") != 0) { free(h); return nullptr; }
    if (hipMemcpy(d, h, n * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        fprintf(stderr, "fortis: copying packed conv weights to the device failed\n");
        fortis_dev_free(d);
        free(h);
        return nullptr;
    }
    free(h);
    if (nfloats) *nfloats = n;
    return d;
}

// The same packing on the device, for callers that hold raw weights in device memory and give them anew with
// every call (the runtime-tier conv entries): W[F][C][T] -> a buffer of the library (one for all shapes,
// grown on demand and kept; launches on the library's stream run one after the other).
__global__ void conv_pack_kernel(const float* __restrict__ W, float* __restrict__ P, long F, long C, int T, int FT, int CC, long nch,
                                 long n)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int NCP = CC / 2;
    long r = idx;
    const int fl = (int)(r % FT); r /= FT;
    const int hh = (int)(r % 2); r /= 2;
    const int t = (int)(r % T); r /= T;
    const int cp = (int)(r % NCP); r /= NCP;
    const long ch = r % nch, fgi = r / nch;
    const long f = fgi * FT + fl, c = ch * CC + cp * 2 + hh;
    P[idx] = (f < F && c < C) ? W[(f * C + c) * T + t] : 0.f;
}

const float* fortis_conv_mfma_pack_dev(const float* dW, long F, long C, int T, hipStream_t st, int kg)
{
    float*& buf = g_pack;
    size_t& cap = g_pack_cap;
    const long FT = kg > 1 ? 32 : conv_ft(F), CC = cm_cc(T) * kg;
    const long nch = cdiv(C, CC), n = cdiv(F, FT) * nch * (CC / 2) * T * 2 * FT;
    if (g_ws) {
        float* w = ws_take(0, (size_t)n * sizeof(float));
        if (!w) return nullptr;
        g_ws_pack = ((size_t)n * sizeof(float) + 255) & ~(size_t)255;
        hipLaunchKernelGGL(conv_pack_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, st, dW, w, F, C, T, (int)FT, (int)CC, nch, n);
        HIP_OK(hipGetLastError());
        return w;
    }
    if ((size_t)n * sizeof(float) > cap) {
        float* p = nullptr;
        if (fortis_dev_malloc((void**)&p, (size_t)n * sizeof(float), "packed conv weights") != 0) return nullptr;
        buf = p;                                   // an outgrown buffer stays: a captured graph may name it
        cap = (size_t)n * sizeof(float);
    }
    hipLaunchKernelGGL(conv_pack_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, st, dW, buf, F, C, T, (int)FT, (int)CC, nch, n);
    HIP_OK(hipGetLastError());
    return buf;
}

template <int KD, int KS, int MT, int FT, int NX, bool TILE2D, int KG = 1, int POOL = 0>
static int launch_nx(const float* x, const float* wp, float* y, ConvMShape s, const ConvEpi& e, hipStream_t st)
{
    constexpr int T = KD * KS * KS;
    constexpr int CC = cm_cc(T) * KG;
    s.tiles = (int)cdiv(s.plane, MT);
    s.R = MT + (KS == 3 ? 2 * s.P + 2 : 0);
    if (TILE2D) {
        s.tiles_x = (int)cdiv(s.W, 32);
        s.tiles = s.tiles_x * (int)cdiv(s.H, MT / 32);
        s.R = (MT / 32 + 2) * CM_TP;
    }
    s.mP = st_magic((unsigned)s.P); s.mR = st_magic((unsigned)s.R); s.mKR = st_magic((unsigned)(KD * s.R));
    s.mT = st_magic((unsigned)s.tiles); s.mTX = st_magic((unsigned)(TILE2D ? s.tiles_x : 1)); s.mNC = st_magic((unsigned)s.nchunks); s.mPer = st_magic(1u);
    // the kernel's weight buffers are padded to whole rounds of 16-byte stores in its forms with unconditional stores
    constexpr int WCH = CC * T * FT, WCHPAD = (WCH / 4 + CM_THREADS - 1) / CM_THREADS * CM_THREADS * 4;
    constexpr bool four_per_cu = KD == 3 && MT == 128 && FT == 64 && NX <= 8;
    const size_t xchp = (size_t)(((long)CC * KD * s.R + 64) / 64 * 64);
    size_t shmem = (size_t)2 * ((four_per_cu ? WCH : WCHPAD) + xchp) * sizeof(float);
    const size_t shmem_sk = (size_t)2 * ((NX <= 8 ? WCHPAD : WCH) + xchp) * sizeof(float);      // the streamed form's
    if (KG > 1 && shmem < 4 * 16 * 64 * sizeof(float)) shmem = 4 * 16 * 64 * sizeof(float);  // (4 / KG tiles) x KG groups x 16 registers x 64 lanes   // the groups' sums meet in LDS
    if (POOL != 0 && shmem < (size_t)((KG > 1 ? 4 * 16 * 64 : 0) + FT * MT) * sizeof(float)) shmem = (size_t)((KG > 1 ? 4 * 16 * 64 : 0) + FT * MT) * sizeof(float);   // the finished tile, for its 2 x 2 max pool
    if (shmem > 160 * 1024 || shmem_sk > 160 * 1024) return -1;
    static size_t attr = 0;
    if (shmem > attr) {
        HIP_OK(hipFuncSetAttribute((const void*)conv_mfma_kernel<KD, KS, MT, FT, NX, TILE2D, KG, POOL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        if constexpr (KD == 3 && KG == 1 && !POOL && !TILE2D)
            HIP_OK(hipFuncSetAttribute((const void*)conv_mfma_kernel<KD, KS, MT, FT, NX, TILE2D, KG, POOL, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem_sk));
        attr = shmem;
    }
    // A launch that leaves most CUs idle (deep, small images) is split over the input channels: each
    // split writes raw partial sums, a second kernel adds them in order and applies the epilogue.
    const long wgs = (long)s.D * s.tiles * cdiv(s.F, FT);
    s.ksplit = 1;
    s.cbase = s.nchunks; s.cextra = 0;
    if (KG == 1 && !POOL && 2 * wgs < 3 * conv_cus() && s.C >= 32) {
        // volumes aim at three workgroups per CU (their chunks are long: 27 taps), images at one (measured on the
        // UNet levels: a finer split costs more in partial sums than it gains in occupancy)
        long k = cdiv((KD == 3 ? 3L : 1L) * conv_cus(), wgs);
        if (k > s.C / 16) k = s.C / 16;               // at least 16 input channels per split
        if (k > 16) k = 16;
        // slices in chunks, the remainder spread over the first ones: the larger slices are dispatched first
        s.ksplit = (int)k;
        s.cbase = (int)(s.nchunks / k); s.cextra = (int)(s.nchunks % k);
    }
    const long ospatial = (long)s.D * s.H * s.W * (s.mode ? 4 : 1);
    s.osize = (long)(s.mode ? s.F / 4 : s.F) * ospatial;
    if constexpr (KD == 3 && KG == 1 && !POOL && !TILE2D) {
        // Volumes whose tiles do not fill the chip evenly.  Fewer tiles than the chip needs (the launch would be split
        // into whole slices): every tile is streamed, in equal runs of (tile, chunk) items.  More tiles than are
        // resident at once, with a last round that would leave most CUs idle while its few workgroups finish: the
        // full rounds run as they are, in a launch of their own, and only the tiles of the last round are streamed.
        static const int sk_wgs = getenv("FORTIS_CONV_STREAMK") ? atoi(getenv("FORTIS_CONV_STREAMK")) : 2;   // streaming workgroups per CU; 0: off
        if (!s.mode && !e.pool && sk_wgs > 0 && s.C >= 32) {
            const long nfg = cdiv(s.F, FT), ntiles = (long)s.D * s.tiles;
            long tile0 = -1;
            if (s.ksplit > 1) tile0 = 0;
            else if (MT == 128 && FT == 64 && NX <= 8) {                 // the form that runs four workgroups per CU
                const long resident = 4L * conv_cus() / nfg, last = ntiles % resident;
                if (ntiles > resident && last > 0 && 2 * last < resident) tile0 = ntiles - last;
            }
            const long items = tile0 < 0 ? 0 : (ntiles - tile0) * s.nchunks;
            long per = cdiv(items, std::max(1L, (long)sk_wgs * conv_cus() / nfg));
            if (per < 8) per = 8;                                         // at least 16 input channels per run
            if (tile0 >= 0 && per < s.nchunks) {
                const long slots = (s.nchunks - 2 + per) / per + 1;       // a tile's items meet at most this many runs
                s.sk_per = (int)per; s.sk_items = (int)items; s.sk_tile0 = (int)tile0;
                s.mPer = st_magic((unsigned)per);
                s.ksplit = 1;
                s.cbase = s.nchunks; s.cextra = 0;
                s.part = fortis_conv_split_scratch((size_t)slots * nfg * (ntiles - tile0) * MT * FT * sizeof(float));
                if (!s.part) return -1;
                if (tile0 > 0) {
                    hipLaunchKernelGGL((conv_mfma_kernel<KD, KS, MT, FT, NX, TILE2D, KG, POOL>), dim3((unsigned)tile0, (unsigned)nfg, 1), dim3(CM_THREADS), shmem, st, x, wp, y, s, e);
                    HIP_OK(hipGetLastError());
                }
                hipLaunchKernelGGL((conv_mfma_kernel<KD, KS, MT, FT, NX, TILE2D, KG, POOL, true>), dim3((unsigned)cdiv(items, per), (unsigned)nfg, 1), dim3(CM_THREADS), shmem_sk, st, x, wp, y, s, e);
                HIP_OK(hipGetLastError());
                hipLaunchKernelGGL((conv_sk_reduce_kernel<MT, FT>), dim3((unsigned)(ntiles - tile0), (unsigned)nfg, (MT / 32 / (4 / (FT / 32))) * 4 / CM_RQB), dim3(CM_THREADS), 0, st, y, s, e);
                HIP_OK(hipGetLastError());
                return 0;
            }
        }
    }
    if (s.ksplit > 1) {
        s.part = fortis_conv_split_scratch((size_t)s.ksplit * s.osize * sizeof(float));
        if (!s.part) return -1;
    }
    // a shape is refused before anything is launched: -1 always means that nothing ran
    const bool pooled = e.pool != nullptr;
    if (pooled && (s.mode || s.D != 1 || (s.H & 1) || (s.W & 1) || (((uintptr_t)y | (uintptr_t)s.part) & 7))) return -1;   // the plan only asks for it on 2-D convs
    dim3 grid((unsigned)(s.D * s.tiles), (unsigned)cdiv(s.F, FT), (unsigned)s.ksplit);
    hipLaunchKernelGGL((conv_mfma_kernel<KD, KS, MT, FT, NX, TILE2D, KG, POOL>), grid, dim3(CM_THREADS), shmem, st, x, wp, y, s, e);
    HIP_OK(hipGetLastError());
    if (s.ksplit > 1 && pooled) {
        const long n = (long)s.F * (s.H / 2) * (s.W / 2);
        hipLaunchKernelGGL(conv_split_reduce_pool_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, st, s.part, y, e.pool, s.F, s.H, s.W,
                           s.osize, s.ksplit, e);
        HIP_OK(hipGetLastError());
    } else if (s.ksplit > 1) {
        launch_split_reduce(s.part, y, s.osize, ospatial, s.ksplit, e, st);
        HIP_OK(hipGetLastError());
    } else if (pooled && POOL != 1) {
        fortis_launch_maxpool2d(y, e.pool, s.F, s.H, s.W, 2, st);
    }
    return 0;
}

template <int KD, int KS, int MT, int FT>
static int launch(const float* x, const float* wp, float* y, ConvMShape s, const ConvEpi& e, hipStream_t st)
{
    if ((long)cm_cc(KD * KS * KS) * s.D * s.H * s.W >= (1L << 30)) return -1;   // a chunk's byte offsets must fit 32 bits
    if constexpr (KD == 1 && KS == 3) {
        // image at least one tile wide whose width fills its 32-column tiles to 80 % or more: rows of 32
        // columns with a one-pixel border; the staging rounds are a compile-time count
        if (s.W >= 32 && cdiv(s.W, 32) * 32 * 4 <= 5L * s.W && getenv("FORTIS_CONV_LINEAR") == nullptr) {
            constexpr int NX2 = (cm_cc(9) * (MT / 32 + 2) * CM_TP + CM_THREADS - 1) / CM_THREADS;
            // a conv with a 2 x 2 max pool behind it pools its own tiles (even tile height) unless the launch is one
            // that gets split over its input channels, whose reduce kernel pools
            if constexpr ((MT / 32) % 2 == 0) {
                const long wgs = cdiv(s.W, 32) * cdiv(s.H, MT / 32) * cdiv(s.F, FT);
                if (e.pool && !s.mode && !(s.H & 1) && !(s.W & 1) && (wgs >= conv_cus() || s.C < 32))
                    return launch_nx<1, 3, MT, FT, NX2, true, 1, true>(x, wp, y, s, e, st);
            }
            return launch_nx<1, 3, MT, FT, NX2, true>(x, wp, y, s, e, st);
        }
    }
    const long R = MT + (KS == 3 ? 2 * s.P + 2 : 0), xch = (long)cm_cc(KD * KS * KS) * KD * R;
    if (xch > (long)CM_THREADS * CM_NXMAX) return -1;     // run too long to stage
    if constexpr (KD == 3 && MT == 128) {
        // volumes: the staging rounds are paid for in matrix time, so the common widths get their exact count
        if (xch <= CM_THREADS * 5) return launch_nx<KD, KS, MT, FT, 5, false>(x, wp, y, s, e, st);
        if (xch <= CM_THREADS * 6) return launch_nx<KD, KS, MT, FT, 6, false>(x, wp, y, s, e, st);
        if (xch <= CM_THREADS * 7) return launch_nx<KD, KS, MT, FT, 7, false>(x, wp, y, s, e, st);
    }
    return xch <= CM_THREADS * 8 ? launch_nx<KD, KS, MT, FT, 8, false>(x, wp, y, s, e, st) : launch_nx<KD, KS, MT, FT, 16, false>(x, wp, y, s, e, st);
}

// Positions per workgroup: the largest tile that still gives every CU about two workgroups; small images
// (deep UNet levels) take the smallest tile so that the launch spreads over the chip at all.
template <int KD, int KS, int FT>
static int launch_mt(const float* x, const float* wp, float* y, ConvMShape s, const ConvEpi& e, hipStream_t st)
{
    s.P = KS == 3 ? s.W + 1 : s.W;
    s.plane = s.H * s.P;
    s.nchunks = (int)cdiv(s.C, cm_cc(KD * KS * KS));
    const long want = 2L * conv_cus(), groups = (long)s.D * cdiv(s.F, FT);
    constexpr int MTMIN = FT == 64 ? 64 : 128;
    if (KD == 1 && groups * cdiv(s.plane, 256) >= want && launch<KD, KS, 256, FT>(x, wp, y, s, e, st) == 0) return 0;
    // images: 128 positions only if that alone fills the chip (a smaller tile beats a channel split with its
    // reduce kernel); volumes keep 128 positions down to half of that (their chunks are long enough to split)
    if ((KD == 1 ? 1 : 2) * groups * cdiv(s.plane, 128) >= want || MTMIN == 128) return launch<KD, KS, 128, FT>(x, wp, y, s, e, st);
    return launch<KD, KS, MTMIN, FT>(x, wp, y, s, e, st);
}

// kind: 0 conv (KD x KS x KS, pad KS/2), 1 transposed 2x2 stride 2, 2 conv whose input (given at half
// resolution) is read through a nearest x2 upsample; D, H, Wd are always the conv's own input extents.  Returns -1 if the shape is not
// one the MFMA kernel takes (the caller then uses the direct kernel).
int fortis_launch_conv_mfma(const float* x, const float* wp, float* y, long C, long D, long H, long Wd, long F, int KD,
                            int KS, int kind, const ConvEpi& e, hipStream_t st)
{
    if (C * D * H * Wd >= 2147483647L || F * D * H * Wd * (kind == 1 ? 4 : 1) >= 2147483647L) return -1;
    if (KD == 1 && D != 1) return -1;                  // the image kernels take one plane
    ConvMShape s;
    memset(&s, 0, sizeof s);
    s.C = (int)C; s.D = (int)D; s.H = (int)H; s.W = (int)Wd;
    s.F = (int)(kind == 1 ? 4 * F : F);
    s.mode = kind == 1 ? 1 : 0;
    s.ksplit = 1;
    s.ups = kind == 2 ? 1 : 0;
    if (kind == 2 && (KD != 3 || ((D | H | Wd) & 1))) return -1;     // the fused upsample is a form of the volume kernel
    if (e.head_y && !fortis_conv_mfma_head_ok(C, H, Wd, F, KD, KS, e.head_n)) return -1;
    const int kgr = kind == 2 ? 1 : fortis_conv_mfma_kgroups(C, D, H, Wd, s.F, KD, KS, e.pool != nullptr && kind == 0);
    if (kgr == 2) {
        if (KS == 1) {
            s.P = s.W;
            s.plane = s.H * s.P;
            s.nchunks = (int)cdiv(s.C, cm_cc(1) * 2);
            return launch_nx<1, 1, 64, 32, cm_cc(1) * 2 * 64 / CM_THREADS, false, 2>(x, wp, y, s, e, st);
        }
        // 64 x 32 output tiles (3 x 3: two rows of the 32-column tiling), two waves per 32 positions, each taking half of a chunk's channels
        s.P = s.W + 1;
        s.plane = s.H * s.P;
        s.nchunks = (int)cdiv(s.C, cm_cc(9) * 2);
        constexpr int NX2 = (cm_cc(9) * 2 * (64 / 32 + 2) * CM_TP + CM_THREADS - 1) / CM_THREADS;
        if (e.head_y) return e.pool || s.mode || s.F > 32 || e.head_n > 4 ? -1 : launch_nx<1, 3, 64, 32, NX2, true, 2, 2>(x, wp, y, s, e, st);
        if (e.pool && !s.mode && !(s.H & 1) && !(s.W & 1)) return launch_nx<1, 3, 64, 32, NX2, true, 2, 1>(x, wp, y, s, e, st);
        return launch_nx<1, 3, 64, 32, NX2, true, 2>(x, wp, y, s, e, st);
    }
    if (kgr == 4) {
        // one 32 x 32 output tile per workgroup, the four waves share its input channels
        s.P = KS == 3 ? s.W + 1 : s.W;
        s.plane = s.H * s.P;
        s.nchunks = (int)cdiv(s.C, cm_cc(KS * KS) * 4);
        if (KS == 3) {
            constexpr int NX2 = (cm_cc(9) * 4 * (32 / 32 + 2) * CM_TP + CM_THREADS - 1) / CM_THREADS;
            return launch_nx<1, 3, 32, 32, NX2, true, 4>(x, wp, y, s, e, st);
        }
        return launch_nx<1, 1, 32, 32, cm_cc(1) * 4 * 32 / CM_THREADS, false, 4>(x, wp, y, s, e, st);
    }
    const bool thin = conv_ft(s.F) == 32;
    if (kind == 1) {
        if (D != 1) return -1;
        return thin ? launch_mt<1, 1, 32>(x, wp, y, s, e, st) : launch_mt<1, 1, 64>(x, wp, y, s, e, st);
    }
    if (KD == 3 && KS == 3) return thin ? launch_mt<3, 3, 32>(x, wp, y, s, e, st) : launch_mt<3, 3, 64>(x, wp, y, s, e, st);
    if (KD == 1 && KS == 3) return thin ? launch_mt<1, 3, 32>(x, wp, y, s, e, st) : launch_mt<1, 3, 64>(x, wp, y, s, e, st);
    if (KD == 1 && KS == 1) return thin ? launch_mt<1, 1, 32>(x, wp, y, s, e, st) : launch_mt<1, 1, 64>(x, wp, y, s, e, st);
    return -1;
}
