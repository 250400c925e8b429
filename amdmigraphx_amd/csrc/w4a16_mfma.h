// int4 weight-only GEMM for M >= 2 on the matrix cores (included by w4a16.hip inside its anonymous
// namespace).
//
// The shapes are bound by the weight stream (K*N/2 bytes against 2*M*N*K flops), so the weights are
// read exactly once, in the largest contiguous pieces the layout allows, and dequantized in
// registers; activations come from L2.
//
// Work split.  A workgroup owns 16*NT output columns (weight rows n0 ..) for up to 128 rows of A.  It
// has 8 compute waves and one fetch wave.  K is walked in chunks of 2048: every weight row
// contributes 1 KiB to a chunk, fetched by ONE global_load_lds instruction (64 lanes x 16 bytes,
// contiguous in memory) straight into an LDS ring of RING chunks; RING-1 chunks stay in flight.  The
// fetch wave issues all of these and is the only wave whose vector-memory counter they occupy:
// memory operations of a wave complete in order, so a compute wave that issued ring loads would
// have every activation load queue behind a weight fetch still on its way from HBM.  Inside a
// chunk the 16 steps of 128 k are dealt to the compute waves (wave w: steps w and w + 8).  For a step and a 16-column tile, lane
// l = 16*kg + n reads its 16 bytes W[n, 128*t + 32*kg .. +32] from LDS (row pitch 1040 bytes: the 16
// rows of a quarter wave fall into distinct banks), the four dwords are transposed across the wave's
// 16-lane rows (v_permlane32_swap, v_permlane16_swap), and dword j of lane-row kg then holds the 8
// weights k = 128*t + 32*j + 8*kg .. +8: the B operand of the j-th v_mfma_f32_16x16x32_f16.  The
// matching A operand of M-tile i is A[16*i + (l & 15), same 8 k], a 16-byte load; for a given j
// the four lane-rows read 64 contiguous bytes of an activation row.  With NT = 2 one A operand
// feeds two column tiles.  Each wave accumulates its K share in fp32; the 8 partial tiles are added
// through LDS in wave order, so the result does not depend on timing.
//
// Dequantization, two weights per instruction, in natural k order: byte r of a dword (nibbles 2r,
// 2r+1) is copied to bytes 0 and 2 of a register with v_perm_b32; (t & 0x00f0000f) | 0x64006400
// then reads as the halves (1024 + q0, 1024 + 16*q1).  Subtracting (1024 + zp, 1024 + 16*zp) is
// exact, and the packed multiply by (s, s/16) under round-toward-zero forms (q - zp) * s with the
// single truncation of the reference's float -> half store.  s/16 must be a normal half (exponent
// field of s at least 5); a wave that meets a smaller scale unpacks the high nibble separately.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int WL_WAVES   = 8;                     // compute waves; one more wave fetches
constexpr int WL_THREADS = (WL_WAVES + 1) * 64;

MI355_DEVINL void wl_load_to_lds(const uint8_t* g, uint8_t* l)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g),
                                     (__attribute__((address_space(3))) void*)(l), 16, 0, 0);
}

template <int N>
MI355_DEVINL void wl_wait_vmcnt()
{
    static_assert(N >= 0 && N < 64);
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

MI355_DEVINL void wl_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// SIMPLE: one zero point for the tensor and a group size that is a multiple of 128, so a step
// needs one scale and no zero-point loads (the MatMulNBits default); the general form looks both
// up for each 32-k quarter of a step.
template <int MT, int NT, bool SIMPLE>
__global__ __launch_bounds__(WL_THREADS) void w4a16_mfma_kernel(w4_params p)
{
    constexpr int WL_CHUNK_K  = NT >= 4 ? 1024 : 2048; // k per chunk
    constexpr int WL_ROW      = WL_CHUNK_K / 2;        // bytes of one weight row in a chunk
    constexpr int WL_PITCH    = WL_ROW + 16;           // LDS row pitch
    constexpr int SPC         = WL_CHUNK_K / 128;      // steps per chunk
    constexpr int SPW         = SPC / WL_WAVES;        // steps of a chunk per wave: 1 or 2
    constexpr int RING        = NT == 1 ? 4 : 3;
    constexpr int CHUNK_BYTES = 16 * NT * WL_PITCH;
    static_assert(RING * CHUNK_BYTES <= 160 * 1024 && WL_WAVES * NT * MT * 4 * 64 * 4 <= 160 * 1024);
    constexpr int RED_BYTES   = WL_WAVES * NT * MT * 4 * 64 * 4;
    constexpr int LDS_BYTES   = RING * CHUNK_BYTES > RED_BYTES ? RING * CHUNK_BYTES : RED_BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS_BYTES];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl   = lane & 15;
    const int kg   = lane >> 4;
    const int n0   = blockIdx.x * (16 * NT);
    const int kbytes  = p.k >> 1;
    const int groups  = p.k / p.group;
    const int nsteps  = p.k >> 7;
    const int nchunks = (p.k + WL_CHUNK_K - 1) / WL_CHUNK_K;
    // K split over blockIdx.z (p.partial set): this workgroup walks chunks cbase .. cbase + nloc - 1
    // and leaves float sums in partial[blockIdx.z]; every share holds at least one chunk
    const int cbase = p.partial != nullptr ? (int)blockIdx.z * p.chunks_per_share : 0;
    const int nloc  = p.partial != nullptr ? min(p.chunks_per_share, nchunks - cbase) : nchunks;

    // half-precision arithmetic of this wave truncates from here on (MODE.fp_round bits 3:2); the
    // fp32 accumulation of the matrix cores keeps round-to-nearest
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 2, 2), 3" ::: "memory");

    // ---- weight stream: global -> LDS ring ----------------------------------------------------
    // one instruction per weight row; lanes past the end of K in the last chunk stay off
    const uint8_t* wbase = p.w + (int64_t)n0 * kbytes;
    auto issue_chunk     = [&](int cl) {
        uint8_t* slot   = lds + (cl % RING) * CHUNK_BYTES;
        const int c     = cbase + cl;
        const int valid = min(WL_ROW, kbytes - c * WL_ROW);
        if(lane * 16 < valid)
        {
#pragma unroll
            for(int r = 0; r < 16 * NT; r++)
                wl_load_to_lds(wbase + (int64_t)r * kbytes + c * WL_ROW + lane * 16,
                               slot + r * WL_PITCH);
        }
    };

    // ---- per-lane constants ---------------------------------------------------------------------
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    const uint32_t w_lane = nl * WL_PITCH + kg * 16;
    const uint16_t* srow[NT];
    const uint8_t* zrow[NT];
#pragma unroll
    for(int t = 0; t < NT; t++)
    {
        const int n           = n0 + 16 * t + nl;
        srow[t]               = p.scales + (int64_t)n * groups;
        const int zrow_groups = p.zp_mode == MI355_W4_ZP_PACKED ? (groups + 1) / 2 : groups;
        zrow[t] = p.zp_mode == MI355_W4_ZP_SCALAR ? nullptr : p.zp + (int64_t)n * zrow_groups;
    }
    // activation rows of this lane, clamped so that every load is in bounds; rows past M are
    // computed and dropped
    const uint8_t* abase = reinterpret_cast<const uint8_t*>(p.a);
    uint32_t aoff[MT];
#pragma unroll
    for(int i = 0; i < MT; i++)
    {
        int r   = 16 * i + nl;
        r       = r < p.m ? r : p.m - 1;
        aoff[i] = ((uint32_t)r * (uint32_t)p.lda + kg * 8) * 2;
    }

    v4f acc[NT][MT];
#pragma unroll
    for(int t = 0; t < NT; t++)
#pragma unroll
        for(int i = 0; i < MT; i++)
            acc[t][i] = v4f{0.f, 0.f, 0.f, 0.f};

    uint32_t pair_mask = 0x00F0000Fu, lo_mask = 0x000F000Fu, magic = 0x64006400u;
    asm volatile("" : "+v"(pair_mask), "+v"(lo_mask), "+v"(magic));

    // What a step needs from global memory, requested one step ahead so that the latency runs
    // under the previous step (and, for a wave's first step, under the first weight fetch): the
    // scales and zero points of its 32-k quarters and -- with at most two M-tiles, where the registers
    // allow a second set -- its activation operands.
    constexpr int NQ       = SIMPLE ? 1 : 4;
    constexpr bool A_AHEAD = MT <= 2;
    struct step_inputs
    {
        uint16_t sb[NT][NQ];
        uint8_t z[NT][NQ];
        v8h af[A_AHEAD ? 4 : 1][MT];
    };
    // A request is unconditional -- past the end of K it repeats the last step and its result goes
    // unused -- so that the number of loads in flight at any point is known at compile time and a
    // step waits for its own inputs only, not for the request issued after them.
    auto request = [&](step_inputs& in, int step) __attribute__((always_inline)) {
        step = step < nsteps ? step : nsteps - 1;
#pragma unroll
        for(int t = 0; t < NT; t++)
#pragma unroll
            for(int q = 0; q < NQ; q++)
            {
                const int g = (step * 128 + q * 32) / p.group;
                in.sb[t][q] = srow[t][g];
                uint8_t z   = (uint8_t)p.zp_scalar;
                if(!SIMPLE)
                {
                    if(p.zp_mode == MI355_W4_ZP_GROUP)
                        z = zrow[t][g];
                    else if(p.zp_mode == MI355_W4_ZP_PACKED)
                    {
                        const uint8_t zb = zrow[t][g >> 1];
                        z                = (g & 1) ? (zb >> 4) : (zb & 0xf);
                    }
                }
                in.z[t][q] = z;
            }
        if(A_AHEAD)
        {
#pragma unroll
            for(int j = 0; j < 4; j++)
#pragma unroll
                for(int i = 0; i < MT; i++)
                    in.af[A_AHEAD ? j : 0][i] = *reinterpret_cast<const v8h*>(
                        abase + (aoff[i] + (uint32_t)step * 256 + j * 64));
        }
    };

    // one step (128 k) of the workgroup's column tiles
    auto step_body = [&](auto fast_tag, step_inputs& in, int step, uint32_t slot_addr, int s_in_chunk)
                         __attribute__((always_inline)) {
        constexpr bool fast = decltype(fast_tag)::value;
        // without the second register set: all operands of the step up front for up to four
        // M-tiles, per quarter for eight
        constexpr bool A_UPFRONT = !A_AHEAD && MT <= 4;
        v8h af_now[A_UPFRONT ? 4 : 1][MT];
        if(A_UPFRONT)
        {
#pragma unroll
            for(int j = 0; j < 4; j++)
#pragma unroll
                for(int i = 0; i < MT; i++)
                    af_now[A_UPFRONT ? j : 0][i] = *reinterpret_cast<const v8h*>(
                        abase + (aoff[i] + (uint32_t)step * 256 + j * 64));
        }
#pragma unroll
        for(int t = 0; t < NT; t++)
        {
            v4u wv;
            asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                         : "=v"(wv)
                         : "v"(slot_addr + w_lane + (uint32_t)(t * 16 * WL_PITCH + s_in_chunk * 64))
                         : "memory");
            // 4 x 4 transpose of the dwords over the wave's 16-lane rows: afterwards wa[j] of
            // lane-row kg is what lane-row j read as dword kg
            uint32_t wa[4];
            {
                auto s02 = __builtin_amdgcn_permlane32_swap(wv.x, wv.z, false, false);
                auto s13 = __builtin_amdgcn_permlane32_swap(wv.y, wv.w, false, false);
                auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
                auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
                wa[0]    = t01[0];
                wa[1]    = t01[1];
                wa[2]    = t23[0];
                wa[3]    = t23[1];
            }
            // scale and zero point as packed constants: (s, s/16) and (1024 + zp, 1024 + 16*zp) for
            // the two-nibbles-at-once form, (s, s) and (1024 + zp, 1024 + zp) otherwise
            h2 zoff = {}, scv = {};
            auto constants = [&](uint32_t sb, uint32_t z) {
                const uint32_t zhi = fast ? (z << 4) : z;
                const uint32_t shi = fast ? sb - (4u << 10) : sb;
                zoff = __builtin_bit_cast(h2, (0x6400u | z) | ((0x6400u | zhi) << 16));
                scv  = __builtin_bit_cast(h2, sb | (shi << 16));
            };
            if(SIMPLE)
                constants(in.sb[t][0], in.z[t][0]);
#pragma unroll
            for(int j = 0; j < 4; j++)
            {
                if(!SIMPLE)
                    constants(in.sb[t][SIMPLE ? 0 : j], in.z[t][SIMPLE ? 0 : j]);
                // B operand: the 8 weights k = 128*step + 32*j + 8*kg .. +8 of column n
                h2 x[4];
#pragma unroll
                for(int r = 0; r < 4; r++)
                {
                    const uint32_t sel = 0x0c000c00u | (uint32_t)r | ((uint32_t)r << 16);
                    const uint32_t tb  = __builtin_amdgcn_perm(wa[j], wa[j], sel);
                    if(fast)
                        x[r] = __builtin_bit_cast(h2, and_or(tb, pair_mask, magic));
                    else
                        x[r] = __builtin_bit_cast(
                            h2, and_or((tb & 0xfu) | ((tb >> 4) & 0x000f0000u), lo_mask, magic));
                }
#pragma unroll
                for(int r = 0; r < 4; r++)
                    x[r] = x[r] - zoff;
#pragma unroll
                for(int r = 0; r < 4; r++)
                    x[r] = x[r] * scv;
                // the four packed registers are the operand as they stand
                const v8h bfrag = __builtin_bit_cast(v8h, v4u{__builtin_bit_cast(uint32_t, x[0]),
                                                               __builtin_bit_cast(uint32_t, x[1]),
                                                               __builtin_bit_cast(uint32_t, x[2]),
                                                               __builtin_bit_cast(uint32_t, x[3])});
                if(!A_AHEAD && !A_UPFRONT)
                {
#pragma unroll
                    for(int i = 0; i < MT; i++)
                        af_now[0][i] = *reinterpret_cast<const v8h*>(
                            abase + (aoff[i] + (uint32_t)step * 256 + j * 64));
                }
#pragma unroll
                for(int i = 0; i < MT; i++)
                {
                    const v8h a = A_AHEAD ? in.af[A_AHEAD ? j : 0][i]
                                          : af_now[A_UPFRONT ? j : 0][i];
                    acc[t][i]   = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bfrag, acc[t][i], 0, 0, 0);
                }
            }
        }
    };

    // The two-nibbles-at-once form needs s/16 to be a normal half for every scale of the step; the
    // choice is made once per step and is wave-uniform, so the inner loops carry no branch.  The
    // separate-nibble form is right for any scale.
    auto do_step = [&](step_inputs& in, int step, uint32_t slot_addr, int s_in_chunk) __attribute__((always_inline)) {
        bool ok = true;
#pragma unroll
        for(int t = 0; t < NT; t++)
#pragma unroll
            for(int q = 0; q < NQ; q++)
            {
                const uint32_t sexp = ((uint32_t)in.sb[t][q] >> 10) & 0x1fu;
                ok                  = ok && sexp >= 5 && sexp <= 30;
            }
        if(__builtin_amdgcn_ballot_w64(ok) == __builtin_amdgcn_ballot_w64(true))
            step_body(std::true_type{}, in, step, slot_addr, s_in_chunk);
        else
            step_body(std::false_type{}, in, step, slot_addr, s_in_chunk);
    };

    // ---- main loop ------------------------------------------------------------------------------
    // Barrier c (one per chunk) says: chunk c has landed, and every compute wave is done with chunk
    // c - 1, whose ring slot the next fetch overwrites.  The fetch wave issues 16*NT loads per chunk;
    // they complete in order, so "at most (RING-2) chunks' worth outstanding" means chunk c is in.
    const bool fetcher = wave == WL_WAVES;
    if(fetcher)
    {
#pragma unroll
        for(int c = 0; c < RING - 1; c++)
            if(c < nloc)
                issue_chunk(c);
        for(int c = 0; c < nloc; c++)
        {
            // (the counter holds at most 63: waiting for one load more than needed is harmless)
            constexpr int AHEAD = (RING - 2) * 16 * NT;
            if(c + RING - 2 < nloc)
                wl_wait_vmcnt<(AHEAD < 63 ? AHEAD : 63)>();
            else
                wl_wait_vmcnt<0>();
            wl_barrier();
            if(c + RING - 1 < nloc)
                issue_chunk(c + RING - 1);
        }
    }
    else
    {
        // this wave's steps: step-in-chunk wave (and wave + 8 where a chunk has 16 steps) of every
        // chunk; two input sets alternate from step to step
        step_inputs in[2];
        request(in[0], cbase * SPC + wave);
        if constexpr(SPW == 2)
        {
            for(int c = 0; c < nloc; c++)
            {
                wl_barrier();
                const uint32_t slot_addr = lds0 + (c % RING) * CHUNK_BYTES;
                const int step0          = (cbase + c) * SPC + wave;
                request(in[1], step0 + WL_WAVES);
                if(step0 < nsteps)
                    do_step(in[0], step0, slot_addr, wave);
                request(in[0], step0 + SPC);
                if(step0 + WL_WAVES < nsteps)
                    do_step(in[1], step0 + WL_WAVES, slot_addr, wave + WL_WAVES);
            }
        }
        else
        {
            for(int c = 0; c < nloc; c += 2)
            {
                wl_barrier();
                const int step0 = (cbase + c) * SPC + wave;
                request(in[1], step0 + SPC);
                if(step0 < nsteps)
                    do_step(in[0], step0, lds0 + (c % RING) * CHUNK_BYTES, wave);
                if(c + 1 < nloc)
                {
                    wl_barrier();
                    request(in[0], step0 + 2 * SPC);
                    if(step0 + SPC < nsteps)
                        do_step(in[1], step0 + SPC, lds0 + ((c + 1) % RING) * CHUNK_BYTES, wave);
                }
            }
        }
    }

    // ---- add the waves' partial tiles in wave order ------------------------------------------
    wl_barrier(); // every chunk has been read: the ring's memory becomes the reduction buffer
    float* red = reinterpret_cast<float*>(lds);
    if(!fetcher)
    {
#pragma unroll
        for(int t = 0; t < NT; t++)
#pragma unroll
            for(int i = 0; i < MT; i++)
#pragma unroll
                for(int r = 0; r < 4; r++)
                    red[((wave * NT + t) * MT * 4 + i * 4 + r) * 64 + lane] = acc[t][i][r];
    }
    __syncthreads();
    for(int idx = tid; idx < NT * MT * 4 * 64; idx += WL_THREADS)
    {
        const int l   = idx & 63;
        const int tir = idx >> 6; // (t * MT + i) * 4 + r
        float s       = 0.f;
#pragma unroll
        for(int w = 0; w < WL_WAVES; w++)
            s += red[(w * NT * MT * 4 + tir) * 64 + l];
        // accumulator register r of lane l is D[4*(l >> 4) + r][l & 15]
        const int t = tir / (MT * 4);
        const int i = (tir >> 2) % MT;
        const int m = 16 * i + 4 * (l >> 4) + (tir & 3);
        if(m >= p.m)
            continue;
        if(p.partial != nullptr)
            p.partial[((int64_t)blockIdx.z * p.m + m) * p.n + n0 + 16 * t + (l & 15)] = s;
        else
            p.out[(int64_t)m * p.ldc + n0 + 16 * t + (l & 15)] = f32_to_half_rtz(s);
    }
}

// out = half(sum of the shares' float partial sums), 4 columns per thread, shares added in order
__global__ __launch_bounds__(256) void w4a16_reduce_kernel(const float* partial, uint16_t* out, int m, int n,
                                                            int64_t ldc, int shares)
{
    const int64_t mn = (int64_t)m * n;
    const int64_t e  = 4 * ((int64_t)blockIdx.x * 256 + threadIdx.x);
    if(e >= mn)
        return;
    v4f sum = *reinterpret_cast<const v4f*>(partial + e);
    for(int z = 1; z < shares; z++)
        sum += *reinterpret_cast<const v4f*>(partial + (int64_t)z * mn + e);
    uint16_t* o = out + (e / n) * ldc + (e % n);
#pragma unroll
    for(int r = 0; r < 4; r++)
        o[r] = f32_to_half_rtz(sum[r]);
}

int launch_w4a16_reduce(const w4_params& p, int shares, hipStream_t s)
{
    const int64_t quads = (int64_t)p.m * p.n / 4;
    hipLaunchKernelGGL(w4a16_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, p.partial, p.out,
                       p.m, p.n, p.ldc, shares);
    return mi355_launch_status();
}

// shares of K for the widest column tile: one workgroup per CU, at least one chunk per share.
// The second kernel costs 3-4 us, which the split only wins back with few column tiles and a
// long K (measured at 16 and 32 rows: K = 14336, N = 4096 gains, 4096 x 4096 and 8192 x 8192 do
// not).
template <int NT>
int mfma_gemm_shares(int n, int k)
{
    constexpr int chunk_k = NT >= 4 ? 1024 : 2048;
    const int tiles       = n / (16 * NT);
    const int nchunks     = (k + chunk_k - 1) / chunk_k;
    if(n % (16 * NT) != 0 || n % 4 != 0 || tiles > 64 || nchunks < 8)
        return 1;
    return max(1, min((256 + tiles - 1) / tiles, nchunks));
}

bool mfma_gemm_supported(const w4_params& p)
{
    // lane offsets are 32-bit; the ring loads move whole 16-byte pieces of a packed row
    return p.n % 16 == 0 && p.k % 128 == 0 && p.m >= 1 && (int64_t)p.n * p.k / 2 < (1ll << 31) &&
           (int64_t)p.m * p.lda * 2 < (1ll << 31);
}

template <int MT, int NT, bool SIMPLE>
int launch_mfma_variant(const w4_params& p0, hipStream_t s)
{
    w4_params p = p0;
    p.partial   = nullptr;
    hipLaunchKernelGGL((w4a16_mfma_kernel<MT, NT, SIMPLE>), dim3(p.n / (16 * NT)), dim3(WL_THREADS), 0, s, p);
    return mi355_launch_status();
}

// the widest tile with K split over `shares` workgroups, then the sum of their partial tiles
template <int MT, int NT, bool SIMPLE>
int launch_mfma_split(const w4_params& p0, int shares, hipStream_t s)
{
    constexpr int chunk_k = NT >= 4 ? 1024 : 2048;
    w4_params p           = p0;
    const int nchunks     = (p.k + chunk_k - 1) / chunk_k;
    p.chunks_per_share    = (nchunks + shares - 1) / shares;
    const int z           = (nchunks + p.chunks_per_share - 1) / p.chunks_per_share;
    hipLaunchKernelGGL((w4a16_mfma_kernel<MT, NT, SIMPLE>), dim3(p.n / (16 * NT), 1, z), dim3(WL_THREADS), 0, s, p);
    return launch_w4a16_reduce(p, z, s);
}

// Every workgroup reads all of A's rows once, from L2: M*K*2 bytes per workgroup against the
// 8*NT*K bytes of weights it owns, so the activations are most of what a CU pulls in unless a
// workgroup's column tile is wide.  The widest tile (NT_MAX column tiles, as the registers allow)
// that still leaves about one workgroup per CU is taken.
template <int MT, int NT_MAX, bool SIMPLE>
int launch_mfma_tiles(const w4_params& p, hipStream_t s)
{
    constexpr int64_t enough = 200;
    if constexpr(NT_MAX >= 2)
    {
        // with room for partial sums: the widest tile (fewest re-reads of A) and K split
        const int shares = mfma_gemm_shares<NT_MAX>(p.n, p.k);
        if(p.partial != nullptr && shares > 1 && (size_t)shares * p.m * p.n * 4 <= p.partial_bytes)
            return launch_mfma_split<MT, NT_MAX, SIMPLE>(p, shares, s);
    }
    if constexpr(NT_MAX >= 4)
    {
        if(p.n % 64 == 0 && p.n / 64 >= enough)
            return launch_mfma_variant<MT, 4, SIMPLE>(p, s);
    }
    if constexpr(NT_MAX >= 2)
    {
        if(p.n % 32 == 0 && p.n / 32 >= enough)
            return launch_mfma_variant<MT, 2, SIMPLE>(p, s);
    }
    return launch_mfma_variant<MT, 1, SIMPLE>(p, s);
}

bool tile_gemm_supported(const w4_params& p);
int launch_tile_gemm(const w4_params& p, hipStream_t s);

// M rows in chunks of at most 128
int launch_mfma_gemm(const w4_params& p0, hipStream_t s)
{
    // the tile kernel takes any number of rows in one launch (64 per workgroup)
    if(tile_gemm_supported(p0))
        return launch_tile_gemm(p0, s);
    for(int m0 = 0; m0 < p0.m; m0 += 128)
    {
        w4_params p = p0;
        p.a         = p0.a + (int64_t)m0 * p0.lda;
        p.out       = p0.out + (int64_t)m0 * p0.ldc;
        p.m         = p0.m - m0 < 128 ? p0.m - m0 : 128;
        int st;
        if(tile_gemm_supported(p))
        {
            st = launch_tile_gemm(p, s);
            if(st != MI355_OK)
                return st;
            continue;
        }
        // (the general zero-point form keeps more per-step state and has room for narrower tiles)
        const bool simple = p.zp_mode == MI355_W4_ZP_SCALAR && (p.group & 127) == 0;
        if(p.m <= 16)
            st = simple ? launch_mfma_tiles<1, 4, true>(p, s) : launch_mfma_tiles<1, 2, false>(p, s);
        else if(p.m <= 32)
            st = simple ? launch_mfma_tiles<2, 4, true>(p, s) : launch_mfma_tiles<2, 2, false>(p, s);
        else if(p.m <= 64)
            st = simple ? launch_mfma_tiles<4, 2, true>(p, s) : launch_mfma_tiles<4, 1, false>(p, s);
        else
            st = simple ? launch_mfma_tiles<8, 1, true>(p, s) : launch_mfma_tiles<8, 1, false>(p, s);
        if(st != MI355_OK)
            return st;
    }
    return MI355_OK;
}
