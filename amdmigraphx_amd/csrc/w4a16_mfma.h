// int4 weight-only GEMM for 2 <= M <= 128 on the matrix cores (included by w4a16.hip inside its
// anonymous namespace).
//
// The shapes are still bound by the weight stream (K*N/2 bytes against 2*M*N*K flops), so the
// weights are read once, in 16-byte loads, straight into the register layout the MFMA wants and
// dequantized there; activations come from L2.
//
// Work split: a workgroup owns 16 output columns (weight rows n0 .. n0+15) for all M rows.  Its
// NW waves split K between them in steps of 128 (runs of WM_DEPTH consecutive steps per wave).  In
// a step, lane l = 16*kg + n loads the 32 weights W[n0+n, 128*t + 32*kg .. +32] with one 16-byte
// load, so a wave instruction reads 64 contiguous bytes of each of its 16 rows.  The four dwords
// are then transposed across the four 16-lane rows of the wave (v_permlane32_swap,
// v_permlane16_swap: four instructions), after which dword j of lane-row kg holds the 8 weights
// k = 128*t + 32*j + 8*kg .. +8: the B operand of the j-th v_mfma_f32_16x16x32_f16.  The matching
// A operand of M-tile i is A[16*i + (l & 15), same 8 k]: for a given j the four lane-rows read 64
// contiguous bytes of an activation row, so these loads use whole cache-line halves as well.
// Each wave accumulates its K share in fp32; the NW partial tiles are added through LDS in wave
// order, so the result does not depend on timing.
//
// Dequantization, two weights per instruction, in natural k order (the A operand needs no
// shuffle): byte r of a dword (nibbles 2r, 2r+1) is copied to bytes 0 and 2 of a register with
// v_perm_b32; (t & 0x00f0000f) | 0x64006400 then reads as the halves (1024 + q0, 1024 + 16*q1).
// Subtracting (1024 + zp, 1024 + 16*zp) is exact, and the packed multiply by (s, s/16) under
// round-toward-zero forms (q - zp) * s with the single truncation of the reference's
// float -> half store.  s/16 must be a normal half (exponent field of s at least 5); a wave that
// meets a smaller scale unpacks the high nibble separately instead.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int WM_DEPTH = 4; // weight loads in flight per lane

// SIMPLE: one zero point for the tensor and a group size that is a multiple of 128, so a step
// needs one scale and no zero-point loads (the MatMulNBits default); the general form looks
// both up for each 32-k quarter of a step.
template <int MT, int NW, bool SIMPLE>
__global__ __launch_bounds__(NW * 64) void w4a16_mfma_kernel(w4_params p)
{
    __shared__ float red[NW][MT * 4][64];
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl   = lane & 15;
    const int kg   = lane >> 4;
    const int n0   = blockIdx.x * 16;
    const int n    = n0 + nl;
    const int kbytes = p.k >> 1;
    const int groups = p.k / p.group;
    const int nsteps = p.k >> 7;

    // half-precision arithmetic of this wave truncates from here on (MODE.fp_round bits 3:2);
    // the fp32 accumulation of the matrix cores keeps round-to-nearest
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 2, 2), 3" ::: "memory");

    // uniform base pointers plus 32-bit lane offsets keep the address arithmetic short
    const uint8_t* wbase  = p.w;
    const uint32_t woff   = (uint32_t)n * (uint32_t)kbytes + kg * 16;
    const uint16_t* srow  = p.scales + (int64_t)n * groups;
    const int zrow_groups = p.zp_mode == MI355_W4_ZP_PACKED ? (groups + 1) / 2 : groups;
    const uint8_t* zrow   = p.zp_mode == MI355_W4_ZP_SCALAR ? nullptr : p.zp + (int64_t)n * zrow_groups;

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

    v4f acc[MT];
#pragma unroll
    for(int i = 0; i < MT; i++)
        acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

    v4u wbuf[WM_DEPTH];
    uint16_t sbuf[WM_DEPTH][4];
    uint8_t zbuf[WM_DEPTH][4];
    // the four 32-k quarters of a step share one scale when the group size is a multiple of 128
    const bool one_group = SIMPLE || (p.group & 127) == 0;
    auto step_of = [&](int round, int u) { return (round * NW + wave) * WM_DEPTH + u; };
    auto issue = [&](int slot, int t) {
        if(t < nsteps)
        {
            wbuf[slot] = __builtin_nontemporal_load(
                reinterpret_cast<const v4u*>(wbase + (woff + (uint32_t)t * 64)));
#pragma unroll
            for(int j = 0; j < 4; j++)
            {
                if(j > 0 && one_group)
                {
                    sbuf[slot][j] = sbuf[slot][0];
                    zbuf[slot][j] = zbuf[slot][0];
                    continue;
                }
                const int g   = (t * 128 + j * 32) / p.group;
                sbuf[slot][j] = srow[g];
                uint8_t z     = (uint8_t)p.zp_scalar;
                if(SIMPLE)
                {
                }
                else if(p.zp_mode == MI355_W4_ZP_GROUP)
                    z = zrow[g];
                else if(p.zp_mode == MI355_W4_ZP_PACKED)
                {
                    const uint8_t zb = zrow[g >> 1];
                    z                = (g & 1) ? (zb >> 4) : (zb & 0xf);
                }
                zbuf[slot][j] = z;
            }
        }
    };
#pragma unroll
    for(int u = 0; u < WM_DEPTH; u++)
        issue(u, step_of(0, u));

    uint32_t pair_mask = 0x00F0000Fu, lo_mask = 0x000F000Fu, magic = 0x64006400u;
    asm volatile("" : "+v"(pair_mask), "+v"(lo_mask), "+v"(magic));

    // Activation operands.  Up to two M-tiles: the operands of the wave's next step are loaded
    // while the current step is computed (two register sets).  More tiles: all operands of a
    // step are requested before its first MFMA, so the loads overlap one another.
    constexpr bool A_AHEAD = MT <= 2;
    v8h abuf[A_AHEAD ? 2 : 1][4][MT];
    auto load_a = [&](int set, int t) {
        if(t < nsteps)
        {
#pragma unroll
            for(int j = 0; j < 4; j++)
#pragma unroll
                for(int i = 0; i < MT; i++)
                    abuf[set][j][i] = *reinterpret_cast<const v8h*>(
                        abase + (aoff[i] + (uint32_t)t * 256 + j * 64));
        }
    };
    if(A_AHEAD)
        load_a(0, step_of(0, 0));

    auto consume = [&](int slot, int t, int t_next) {
        const int set = A_AHEAD ? (slot & 1) : 0;
        if(A_AHEAD)
            load_a(set ^ 1, t_next);
        else
            load_a(0, t);
        // 4 x 4 transpose of the dwords over the wave's 16-lane rows: afterwards wa[j] of
        // lane-row kg is what lane-row j loaded as dword kg
        uint32_t wa[4] = {wbuf[slot].x, wbuf[slot].y, wbuf[slot].z, wbuf[slot].w};
        {
            auto s02 = __builtin_amdgcn_permlane32_swap(wa[0], wa[2], false, false);
            auto s13 = __builtin_amdgcn_permlane32_swap(wa[1], wa[3], false, false);
            auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
            auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
            wa[0]    = t01[0];
            wa[1]    = t01[1];
            wa[2]    = t23[0];
            wa[3]    = t23[1];
        }
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            const uint32_t sb   = sbuf[slot][j];
            const uint32_t z    = zbuf[slot][j];
            const uint32_t sexp = (sb >> 10) & 0x1fu;
            // wave-uniform choice; the separate-nibble form is right for any scale
            const bool fast = __builtin_amdgcn_ballot_w64(sexp >= 5 && sexp <= 30) == ~0ull;
            h2 zoff, scv;
            if(fast)
            {
                zoff = __builtin_bit_cast(h2, (0x6400u | z) | ((0x6400u | (z << 4)) << 16));
                scv  = __builtin_bit_cast(h2, sb | ((sb - (4u << 10)) << 16));
            }
            else
            {
                zoff = __builtin_bit_cast(h2, (0x6400u | z) | ((0x6400u | z) << 16));
                scv  = __builtin_bit_cast(h2, sb | (sb << 16));
            }
            // B operand: the 8 weights k = 128*t + 32*j + 8*kg .. +8 of column n
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
            v8h bfrag;
#pragma unroll
            for(int r = 0; r < 4; r++)
            {
                bfrag[2 * r]     = x[r][0];
                bfrag[2 * r + 1] = x[r][1];
            }
#pragma unroll
            for(int i = 0; i < MT; i++)
            {
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(abuf[set][j][i], bfrag, acc[i], 0, 0, 0);
            }
        }
    };

    const int rounds = (nsteps + NW * WM_DEPTH - 1) / (NW * WM_DEPTH);
    for(int round = 0; round < rounds; round++)
    {
#pragma unroll
        for(int u = 0; u < WM_DEPTH; u++)
        {
            const int tt = step_of(round, u);
            if(tt < nsteps)
            {
                consume(u, tt, u + 1 < WM_DEPTH ? step_of(round, u + 1) : step_of(round + 1, 0));
                issue(u, step_of(round + 1, u));
            }
        }
    }

    // add the waves' partial tiles in wave order
#pragma unroll
    for(int i = 0; i < MT; i++)
#pragma unroll
        for(int r = 0; r < 4; r++)
            red[wave][i * 4 + r][lane] = acc[i][r];
    __syncthreads();
    for(int idx = tid; idx < MT * 4 * 64; idx += NW * 64)
    {
        const int l  = idx & 63;
        const int ir = idx >> 6;
        float s      = 0.f;
#pragma unroll
        for(int w = 0; w < NW; w++)
            s += red[w][ir][l];
        // accumulator register r of lane l is D[4*(l >> 4) + r][l & 15]
        const int m = 16 * (ir >> 2) + 4 * (l >> 4) + (ir & 3);
        if(m < p.m)
            p.out[(int64_t)m * p.ldc + n0 + (l & 15)] = f32_to_half_rtz(s);
    }
}

bool mfma_gemm_supported(const w4_params& p)
{
    // lane offsets are 32-bit
    return p.n % 16 == 0 && p.k % 128 == 0 && p.m >= 1 && (int64_t)p.n * p.k / 2 < (1ll << 31) &&
           (int64_t)p.m * p.lda * 2 < (1ll << 31);
}

template <int MT>
int launch_mfma_tiles(const w4_params& p, hipStream_t s)
{
    const int grid = p.n / 16;
    // few column tiles: more waves per workgroup keep enough weight loads in flight
    const bool simple = p.zp_mode == MI355_W4_ZP_SCALAR && (p.group & 127) == 0;
    if constexpr(MT == 1)
    {
        if(grid < 512 && (p.k >> 7) >= 32 && simple)
        {
            hipLaunchKernelGGL((w4a16_mfma_kernel<MT, 16, true>), dim3(grid), dim3(1024), 0, s, p);
            return mi355_launch_status();
        }
    }
    if(simple)
        hipLaunchKernelGGL((w4a16_mfma_kernel<MT, 8, true>), dim3(grid), dim3(512), 0, s, p);
    else
        hipLaunchKernelGGL((w4a16_mfma_kernel<MT, 8, false>), dim3(grid), dim3(512), 0, s, p);
    return mi355_launch_status();
}

// M rows in chunks of at most 128
int launch_mfma_gemm(const w4_params& p0, hipStream_t s)
{
    for(int m0 = 0; m0 < p0.m; m0 += 128)
    {
        w4_params p = p0;
        p.a         = p0.a + (int64_t)m0 * p0.lda;
        p.out       = p0.out + (int64_t)m0 * p0.ldc;
        p.m         = p0.m - m0 < 128 ? p0.m - m0 : 128;
        int st;
        if(p.m <= 16)
            st = launch_mfma_tiles<1>(p, s);
        else if(p.m <= 32)
            st = launch_mfma_tiles<2>(p, s);
        else if(p.m <= 64)
            st = launch_mfma_tiles<4>(p, s);
        else
            st = launch_mfma_tiles<8>(p, s);
        if(st != MI355_OK)
            return st;
    }
    return MI355_OK;
}
