// int4 weight-only GEMM for more than 32 rows of A (included by w4a16.hip inside its anonymous
// namespace, after w4a16_mfma.h whose helpers it uses).
//
// With many rows the activations, not the weights, are most of what a workgroup pulls in: a
// workgroup that owns a strip of columns reads all of A once, so the strip has to be wide and the
// activations have to be shared by the waves.  Here a workgroup owns a 64 x 128 tile of the output
// (16*MT rows, MT <= 4).  Its 8 compute waves split the 128 columns (wave w: weight rows n0 + 16*w ..
// +16) and all walk K together in steps of 128; one more wave fetches.  K is cut into chunks of 256:
// a chunk's 128 x 128 bytes of packed weights and 64 x 512 bytes of activations go straight into an
// LDS ring of three slots with global_load_lds (48 instructions of 1 KiB per chunk), two chunks in
// flight while one is consumed.  Every wave reads the whole activation tile from LDS and only its
// own weight rows, so nothing a compute wave needs for the matrix cores comes from global memory:
// its only global loads are one scale (and zero point) per column and step, requested a step ahead.
//
// LDS layout.  A global_load_lds instruction writes 64 consecutive 16-byte pieces, but each lane
// chooses the global address it loads from, so the layout is a permutation of pieces chosen for the
// readers: piece p of weight row r sits at r*8 + (p ^ ((r >> 1) & 7)), piece p (of 32) of activation
// row m at m*32 + (p ^ (m & 15)).  A 16-lane quarter wave reading one piece of 16 consecutive rows
// then touches 16 different 16-byte bank groups, in both arrays.
//
// Per step a wave reads its 16 x 64 bytes of weights, transposes and dequantizes them exactly like
// the K-split kernel (same instructions, same rounding), and for each 32-k quarter multiplies the
// B operand into the MT accumulators with the A operands of that quarter, which were requested from
// LDS one quarter earlier.  The accumulators are the final sums: no reduction across waves.
constexpr int TL_CK   = 256; // k per chunk
constexpr int TL_BN   = 128; // columns per workgroup
constexpr int TL_RING = 3;

// 16-byte LDS reads whose result is not waited for here: the destination is written when the data
// returns, so it is marked early-clobber (it must not share a register with the address)
template <int OFFSET>
MI355_DEVINL void tl_lds_read(v8h& d, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(d) : "v"(addr), "n"(OFFSET));
}

template <int MT, int... I>
MI355_DEVINL void tl_lds_read_tiles(v8h (&af)[MT], uint32_t addr, std::integer_sequence<int, I...>)
{
    (tl_lds_read<I * 8192>(af[I], addr), ...);
}

template <int MT, bool SIMPLE>
__global__ __launch_bounds__(WL_THREADS) void w4a16_tile_kernel(w4_params p)
{
    constexpr int BM      = 16 * MT;
    constexpr int W_BYTES = TL_BN * TL_CK / 2;
    constexpr int A_BYTES = BM * TL_CK * 2;
    constexpr int SLOT    = W_BYTES + A_BYTES;
    constexpr int W_INSTR = W_BYTES / 1024;
    constexpr int A_INSTR = A_BYTES / 1024;
    constexpr int PER_CHUNK = W_INSTR + A_INSTR;
    static_assert((TL_RING - 2) * PER_CHUNK < 64 && TL_RING * SLOT <= 160 * 1024);
    __shared__ __attribute__((aligned(1024))) uint8_t lds[TL_RING * SLOT];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl   = lane & 15;
    const int kg   = lane >> 4;
    const int n0   = blockIdx.x * TL_BN;
    const int m0   = blockIdx.y * BM;
    const int kbytes  = p.k >> 1;
    const int groups  = p.k / p.group;
    const int nsteps  = p.k >> 7;
    const int nchunks = (p.k + TL_CK - 1) / TL_CK;
    // K split over blockIdx.z (p.partial set): this workgroup walks chunks cbase .. cbase + nloc - 1
    // and leaves float sums in partial[blockIdx.z]; every share holds at least one chunk
    const int cbase = p.partial != nullptr ? (int)blockIdx.z * p.chunks_per_share : 0;
    const int nloc  = p.partial != nullptr ? min(p.chunks_per_share, nchunks - cbase) : nchunks;

    // half-precision arithmetic of this wave truncates from here on (MODE.fp_round bits 3:2); the
    // fp32 accumulation of the matrix cores keeps round-to-nearest
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 2, 2), 3" ::: "memory");

    const bool fetcher = wave == WL_WAVES;
    if(fetcher)
    {
        // ---- global -> LDS ring -----------------------------------------------------------------
        // weights: instruction t covers rows 8t .. 8t+7, lane l the piece at position l & 7 of row
        // 8t + (l >> 3).  activations: instruction t covers rows 2t, 2t+1, lane l the piece at
        // position l & 31 of row 2t + (l >> 5).  Rows past M repeat the last row; pieces past the end
        // of K (second half of the last chunk when K is an odd multiple of 128) repeat the first
        // half and are not used.
        // All of a lane's source offsets are fixed up to the chunk's position in K, so they are
        // formed once (32-bit: the operands are smaller than 2 GiB) and an instruction costs one add.
        const uint8_t* abytes = reinterpret_cast<const uint8_t*>(p.a);
        uint32_t wsrc[2], asrc[A_INSTR];
        bool w_second[2], a_second[A_INSTR]; // piece lies in the second half (k >= 128) of a chunk
#pragma unroll
        for(int t = 0; t < 2; t++)
        {
            const int r  = 8 * t + (lane >> 3);
            const int pc = (lane & 7) ^ ((r >> 1) & 7);
            wsrc[t]      = (uint32_t)(n0 + (lane >> 3)) * (uint32_t)kbytes + (uint32_t)(pc * 16);
            w_second[t]  = pc >= 4;
        }
#pragma unroll
        for(int t = 0; t < A_INSTR; t++)
        {
            const int m  = 2 * t + (lane >> 5);
            const int pc = (lane & 31) ^ (m & 15);
            int row      = m0 + m;
            row          = row < p.m ? row : p.m - 1;
            asrc[t]      = ((uint32_t)row * (uint32_t)p.lda + (uint32_t)(pc * 8)) * 2;
            a_second[t]  = pc >= 16;
        }
        auto issue_chunk = [&](int cl) {
            uint8_t* slot = lds + (cl % TL_RING) * SLOT;
            const int c   = cbase + cl;
            // only the first half of the last chunk exists when K is an odd multiple of 128
            const bool half = c * TL_CK + 128 >= p.k;
#pragma unroll
            for(int t = 0; t < W_INSTR; t++)
            {
                uint32_t off = wsrc[t & 1] + (uint32_t)(8 * t) * (uint32_t)kbytes + (uint32_t)(c * (TL_CK / 2));
                if(half)
                    off -= w_second[t & 1] ? 64u : 0u;
                wl_load_to_lds(p.w + off, slot + t * 1024);
            }
#pragma unroll
            for(int t = 0; t < A_INSTR; t++)
            {
                uint32_t off = asrc[t] + (uint32_t)(c * TL_CK * 2);
                if(half)
                    off -= a_second[t] ? 256u : 0u;
                wl_load_to_lds(abytes + off, slot + W_BYTES + t * 1024);
            }
        };
        // Barrier c (one per chunk) says: chunk c has landed, and every compute wave is done with
        // chunk c - 1, whose slot the next fetch overwrites.  The loads complete in order, so "at most
        // one chunk's worth outstanding" means chunk c is in.
#pragma unroll
        for(int c = 0; c < TL_RING - 1; c++)
            if(c < nloc)
                issue_chunk(c);
        for(int c = 0; c < nloc; c++)
        {
            if(c + TL_RING - 2 < nloc)
                wl_wait_vmcnt<(TL_RING - 2) * PER_CHUNK>();
            else
                wl_wait_vmcnt<0>();
            wl_barrier();
            if(c + TL_RING - 1 < nloc)
                issue_chunk(c + TL_RING - 1);
        }
        return;
    }

    // ---- compute waves --------------------------------------------------------------------------
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    const int w_row     = 16 * wave + nl;
    uint32_t w_off[2], a_off[4];
#pragma unroll
    for(int s = 0; s < 2; s++)
        w_off[s] = (uint32_t)((w_row * 8 + ((4 * s + kg) ^ ((w_row >> 1) & 7))) * 16);
#pragma unroll
    for(int j = 0; j < 4; j++)
        a_off[j] = (uint32_t)(W_BYTES + (nl * 32 + ((4 * j + kg) ^ nl)) * 16);

    const int n           = n0 + w_row;
    const uint16_t* srow  = p.scales + (int64_t)n * groups;
    const int zrow_groups = p.zp_mode == MI355_W4_ZP_PACKED ? (groups + 1) / 2 : groups;
    const uint8_t* zrow   = p.zp_mode == MI355_W4_ZP_SCALAR ? nullptr : p.zp + (int64_t)n * zrow_groups;

    v4f acc[MT];
#pragma unroll
    for(int i = 0; i < MT; i++)
        acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

    uint32_t pair_mask = 0x00F0000Fu, lo_mask = 0x000F000Fu, magic = 0x64006400u;
    asm volatile("" : "+v"(pair_mask), "+v"(lo_mask), "+v"(magic));

    // scales and zero points of a step, requested one step ahead; unconditional (past the end of K
    // the last step is repeated) so that the loads in flight can be counted at compile time
    constexpr int NQ = SIMPLE ? 1 : 4;
    struct step_inputs
    {
        uint16_t sb[NQ];
        uint8_t z[NQ];
    };
    auto request = [&](step_inputs& in, int step) __attribute__((always_inline)) {
        step = step < nsteps ? step : nsteps - 1;
#pragma unroll
        for(int q = 0; q < NQ; q++)
        {
            const int g = (step * 128 + q * 32) / p.group;
            in.sb[q]    = srow[g];
            uint8_t z   = (uint8_t)p.zp_scalar;
            if(!SIMPLE)
            {
                if(p.zp_mode == MI355_W4_ZP_GROUP)
                    z = zrow[g];
                else if(p.zp_mode == MI355_W4_ZP_PACKED)
                {
                    const uint8_t zb = zrow[g >> 1];
                    z                = (g & 1) ? (zb >> 4) : (zb & 0xf);
                }
            }
            in.z[q] = z;
        }
    };

    // A operands of quarter j of step-in-chunk s: one 16-byte LDS read per M-tile, not waited for
    auto read_a = [&](v8h (&af)[MT], uint32_t slot_addr, int s, int j) __attribute__((always_inline)) {
        const uint32_t addr = slot_addr + a_off[j] + (uint32_t)(s * 256);
        tl_lds_read_tiles<MT>(af, addr, std::make_integer_sequence<int, MT>{});
    };
    // wait until at most `younger` LDS reads issued after those of af are outstanding; the operands
    // pass through the statement so that their uses cannot move in front of it
    auto wait_a = [&](v8h (&af)[MT], auto younger) __attribute__((always_inline)) {
        constexpr int Y = decltype(younger)::value;
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(af[0]) : "n"(Y));
#pragma unroll
        for(int i = 1; i < MT; i++)
            asm volatile("" : "+v"(af[i]));
    };

    auto step_body = [&](auto fast_tag, step_inputs& in, uint32_t slot_addr, int s) __attribute__((always_inline)) {
        constexpr bool fast = decltype(fast_tag)::value;
        v4u wv;
        v8h af[2][MT];
        asm volatile("ds_read_b128 %0, %1" : "=&v"(wv) : "v"(slot_addr + w_off[s]));
        read_a(af[0], slot_addr, s, 0);
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(wv) : "n"(MT));
        // 4 x 4 transpose of the dwords over the wave's 16-lane rows: afterwards wa[j] of lane-row
        // kg is what lane-row j read as dword kg
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
        // scale and zero point as packed constants: (s, s/16) and (1024 + zp, 1024 + 16*zp) for the
        // two-nibbles-at-once form, (s, s) and (1024 + zp, 1024 + zp) otherwise
        h2 zoff = {}, scv = {};
        auto constants = [&](uint32_t sb, uint32_t z) {
            const uint32_t zhi = fast ? (z << 4) : z;
            const uint32_t shi = fast ? sb - (4u << 10) : sb;
            zoff = __builtin_bit_cast(h2, (0x6400u | z) | ((0x6400u | zhi) << 16));
            scv  = __builtin_bit_cast(h2, sb | (shi << 16));
        };
        if(SIMPLE)
            constants(in.sb[0], in.z[0]);
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            if(j < 3)
                read_a(af[(j + 1) & 1], slot_addr, s, j + 1);
            if(!SIMPLE)
                constants(in.sb[SIMPLE ? 0 : j], in.z[SIMPLE ? 0 : j]);
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
            const v8h bfrag = __builtin_bit_cast(v8h, v4u{__builtin_bit_cast(uint32_t, x[0]),
                                                           __builtin_bit_cast(uint32_t, x[1]),
                                                           __builtin_bit_cast(uint32_t, x[2]),
                                                           __builtin_bit_cast(uint32_t, x[3])});
            if(j < 3)
                wait_a(af[j & 1], std::integral_constant<int, MT>{});
            else
                wait_a(af[j & 1], std::integral_constant<int, 0>{});
#pragma unroll
            for(int i = 0; i < MT; i++)
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[j & 1][i], bfrag, acc[i], 0, 0, 0);
        }
    };
    // The two-nibbles-at-once form needs s/16 to be a normal half for every scale of the step; the
    // choice is made once per step and is wave-uniform.  The separate-nibble form is right for any
    // scale.
    auto do_step = [&](step_inputs& in, uint32_t slot_addr, int s) __attribute__((always_inline)) {
        bool ok = true;
#pragma unroll
        for(int q = 0; q < NQ; q++)
        {
            const uint32_t sexp = ((uint32_t)in.sb[q] >> 10) & 0x1fu;
            ok                  = ok && sexp >= 5 && sexp <= 30;
        }
        if(__builtin_amdgcn_ballot_w64(ok) == __builtin_amdgcn_ballot_w64(true))
            step_body(std::true_type{}, in, slot_addr, s);
        else
            step_body(std::false_type{}, in, slot_addr, s);
    };

    step_inputs in[2];
    request(in[0], 2 * cbase);
    for(int c = 0; c < nloc; c++)
    {
        wl_barrier();
        const uint32_t slot_addr = lds0 + (c % TL_RING) * SLOT;
        const int step           = 2 * (cbase + c);
        request(in[1], step + 1);
        do_step(in[0], slot_addr, 0);
        request(in[0], step + 2);
        if(step + 1 < nsteps)
            do_step(in[1], slot_addr, 1);
    }

    // accumulator register r of lane l is D[4*(l >> 4) + r][l & 15]
#pragma unroll
    for(int i = 0; i < MT; i++)
#pragma unroll
        for(int r = 0; r < 4; r++)
        {
            const int m = m0 + 16 * i + 4 * kg + r;
            if(m >= p.m)
                continue;
            if(p.partial != nullptr)
                p.partial[((int64_t)blockIdx.z * p.m + m) * p.n + n] = acc[i][r];
            else
                p.out[(int64_t)m * p.ldc + n] = f32_to_half_rtz(acc[i][r]);
        }
}

// shares of K for `m` rows: enough workgroups for every CU (a workgroup
// fills one), at least two chunks per share; 1 = no split
int tile_gemm_shares(int m, int n, int k)
{
    const int tiles   = (n / TL_BN) * ((m + 63) / 64);
    const int nchunks = (k + TL_CK - 1) / TL_CK;
    if(tiles > 128 || nchunks < 4)
        return 1;
    int s = (256 + tiles - 1) / tiles;
    s     = min(s, nchunks / 2);
    return max(s, 1);
}

bool tile_gemm_supported(const w4_params& p)
{
    return p.m > 32 && p.n % TL_BN == 0 && mfma_gemm_supported(p);
}

// 64 rows per workgroup
int launch_tile_gemm(const w4_params& p0, hipStream_t s)
{
    w4_params p       = p0;
    const bool simple = p.zp_mode == MI355_W4_ZP_SCALAR && (p.group & 127) == 0;
    dim3 grid((unsigned)(p.n / TL_BN), (unsigned)((p.m + 63) / 64));
    const int shares = tile_gemm_shares(p.m, p.n, p.k);
    float* room      = p0.partial;
    p.partial        = nullptr;
    if(room != nullptr && shares > 1 && (size_t)shares * p.m * p.n * 4 <= p0.partial_bytes)
    {
        const int nchunks  = (p.k + TL_CK - 1) / TL_CK;
        p.chunks_per_share = (nchunks + shares - 1) / shares;
        p.partial          = room;
        grid.z             = (unsigned)((nchunks + p.chunks_per_share - 1) / p.chunks_per_share);
    }
    if(simple)
        hipLaunchKernelGGL((w4a16_tile_kernel<4, true>), grid, dim3(WL_THREADS), 0, s, p);
    else
        hipLaunchKernelGGL((w4a16_tile_kernel<4, false>), grid, dim3(WL_THREADS), 0, s, p);
    if(p.partial != nullptr)
        return launch_w4a16_reduce(p, (int)grid.z, s);
    return mi355_launch_status();
}
