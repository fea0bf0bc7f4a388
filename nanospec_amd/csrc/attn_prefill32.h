// Prompt portions on the 32x32x16 matrix instruction, keys and values loaded straight into LDS (included by
// attn_mfma.hip, which defines AttnParams and the head and page constants).  For head sizes 64 and 128.
//
// A workgroup owns 32 tokens of up to four query heads of one key/value head, one head per wave, as in the 16x16 form
// (attn_prefill_kernel): each block of 32 keys is fetched once per workgroup and shared through LDS, one or two sets of
// four waves walk a tile's keys.  Three things differ.
//
// The matrix instruction.  A SIMD issues one instruction at a time; a 16x16x32 instruction holds the issue port for 8 of
// its 16 cycles and a 32x32x16 instruction for 8 of its 32 (measured with a probe of matrix and vector instructions alone
// and interleaved), so the larger one leaves twice the room for the soft-max's vector instructions beside the same
// arithmetic, and it reads every fragment of the values from LDS once for all 32 tokens instead of once per 16.
//   S^T[key][token] = K[key][:] . Q[token][:]    A = K from LDS (lane: key row lane % 32, channels 8 (lane / 32) .. + 7 of
//                                                a step of 16), B = Q^T from registers (lane: token lane % 32)
//   a lane then holds, for its token, the 16 scores of S rows 8 (r / 4) + 4 (lane / 32) + r % 4, r = 0 .. 15
//   O^T[ch][token] += V^T[ch][key] . P^T[key][token]   A = V^T from LDS (lane: channel lane % 32 of a tile of 32, keys
//                                                8 (lane / 32) .. + 7 of a step of 16), B = P^T = the lane's own weights
// LDS row rho of the keys holds key 16 s + 8 h + 4 b + j of the block for rho = 16 s + 8 b + 4 h + j, so that the weights
// r = 8 s .. 8 s + 7 of a lane are those of keys 16 s + 8 (lane / 32) .. + 7: the eight consecutive keys that one
// 16-byte read of a channel's values brings.  Score r of a lane is key 16 (r / 8) + 8 (lane / 32) + r % 8.
//
// The pipeline.  The keys run one block ahead of the values: a round forms the scores of block j + 1 (matrix
// instructions) beside the soft-max weights of block j (vector instructions on the scores that the round before left),
// then the weighted values of block j.  The two do not depend on each other, so the matrix unit and the vector unit are
// both busy within the one wave.
//
// The loads.  `global_load_lds` writes 16 bytes per lane straight into LDS, the 64 lanes of an instruction side by side:
// no registers hold a block between memory and LDS and no instruction copies it.  Three buffers each for keys and
// values: in round j the keys of block j + 1 and the values of block j are read, the keys of block j + 2 and the values
// of block j + 1 have been asked for a round ago and must have landed when the round ends, and the keys of block j + 3
// and the values of block j + 2 are asked for.  Where a lane's 16 bytes land is fixed by its number, which of the block's
// 16-byte pieces it fetches is free, so the layout in LDS is chosen for the reads:
//   keys:   instruction n of a block (HD / 16 of them, 1 KiB each, 32 bytes apart) holds rows n + (HD / 16) q,
//           q = lane / (HD / 8), and in a row the piece (lane % (HD / 8)) ^ (bit 4 of the row);
//   values: two planes of 16 keys, [channel][16 keys = 32 bytes]; an instruction holds 32 channels of a plane and a
//           lane the half (lane % 2) ^ (bit 4 of the channel) of a channel's 32 bytes.
// A 16-byte LDS read is served for lanes 0-7 and 16-23 together (then 8-15 and 24-31, ...): with these layouts the
// sixteen pieces fall into sixteen different groups of four banks.
// The waits are counted by hand: `s_waitcnt vmcnt(n)` before a plain `s_barrier` lets the loads of the current round stay
// on their way while those of the round before must have landed (the compiler's own barrier would wait for all).
#pragma once

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;

constexpr bool DMA_OK = (HD == 64 || HD == 128) && PS >= 8;  // (other sizes: attn_prefill_kernel)
constexpr int QS = HD / 16;                // matrix instructions per block for the scores
constexpr int CT = HD / 32 > 0 ? HD / 32 : 1;                // tiles of 32 channels of the output
constexpr int NI = HD / 16;                // load instructions per block for the keys; as many for the values
constexpr int IPW = NI / 4 > 0 ? NI / 4 : 1;  // ... per wave
constexpr int KP = HD / 8;                 // 16-byte pieces of a key
constexpr int K_REGION = 1024 + 32;        // bytes from one instruction's keys to the next one's
constexpr int K_BUF = NI * K_REGION;       // a block's keys
constexpr int V_PLANE = HD * 32;           // 16 keys of all channels
constexpr int V_BUF = 2 * V_PLANE;         // a block's values
constexpr int RING = 3;

__device__ __forceinline__ float max_with_other_half(float x) {  // over lanes l and l ^ 32, in both
  const unsigned u = __float_as_uint(x);
  const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(h[0]), __uint_as_float(h[1]));
}

// Wait until at most `n` of this wave's loads are still on their way (and for nothing else).
#define NS_WAIT_LOADS(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

template <int SETS>
__global__ __launch_bounds__(SETS * 256) __attribute__((amdgpu_waves_per_eu(2))) void attn_prefill32_kernel(AttnParams a) {
  if constexpr (DMA_OK) {
    constexpr int SET_BYTES = RING * (K_BUF + V_BUF);
    constexpr int JOIN = CT * 16 + 4;  // floats a lane hands over (a multiple of four: 16-byte LDS accesses)
    constexpr int JOIN_BYTES = SETS == 2 ? 256 * JOIN * 4 : 0;  // what the second set hands to the first: sums, maximum, total
    __shared__ __align__(16) char smem[SETS * SET_BYTES > JOIN_BYTES ? SETS * SET_BYTES : JOIN_BYTES];
    const int half = SETS == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;  // which set of four waves
    char* const kring = smem + half * SET_BYTES;
    char* const vring = kring + RING * K_BUF;
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, h = lane >> 5;  // this lane's token of the tile, and which half of a step's channels or keys it holds
    const int G = a.heads / a.kv_heads;
    const int hblks = (G + 3) / 4;
    const int ny = a.kv_heads * hblks;
    const int split = blockIdx.x % a.splits, ts = blockIdx.x / a.splits;  // the ranges of a tile start together
    // (the key/value head is the fast index of the launch order: see attn_prefill_kernel)
    const int y = ts % ny;
    const int tile = a.n_tiles - 1 - ts / ny;  // the last tiles see the most keys, so they start first
    const int kvh = y / hblks, hin = (y % hblks) * 4 + wave;
    const bool head_ok = hin < G;  // a wave without a head still fetches its share of the keys and values
    const int head = kvh * G + (head_ok ? hin : 0);
    const int4 info = *reinterpret_cast<const int4*>(a.tiles + (size_t)tile * TILE_INTS);
    const int b = __builtin_amdgcn_readfirstlane(info.x), t0 = __builtin_amdgcn_readfirstlane(info.y);
    const int q0 = __builtin_amdgcn_readfirstlane(info.z), n = __builtin_amdgcn_readfirstlane(info.w);
    const int kv_len = __builtin_amdgcn_readfirstlane(a.tiles[(size_t)tile * TILE_INTS + 4]);
    const int* table = a.block_table + (size_t)b * a.table_stride;
    constexpr int psh = __builtin_ctz(PS), pmask = PS - 1;

    const int ti = t0 + c;
    const bool col_ok = ti < n && head_ok;
    const int pos = col_ok ? kv_len - n + ti : -1;
    const int lo = (col_ok && a.window > 0) ? max(0, pos - a.window + 1) : 0;
    // what the tile's tokens see, from the descriptor alone: the same in every wave
    const int first_pos = kv_len - n + t0, last_pos = kv_len - n + min(t0 + 31, n - 1);
    const int whi = last_pos + 1;                                   // keys [wlo, whi) are seen by some token
    const int wlo = a.window > 0 ? max(0, first_pos - a.window + 1) : 0;
    const int full_hi = first_pos;                                  // keys <= full_hi are seen by every token (without a window)
    int tile_kb0 = wlo / 32, tile_kb1 = (whi + 31) / 32;
    if (a.splits > 1) {  // this workgroup's range of the tile's blocks; it may be empty
      const int per = (tile_kb1 - tile_kb0 + a.splits - 1) / a.splits;
      tile_kb0 = min(tile_kb1, tile_kb0 + split * per);
      tile_kb1 = min(tile_kb1, tile_kb0 + per);
    }
    const int steps = SETS == 2 ? (tile_kb1 - tile_kb0 + 1) / 2 : tile_kb1 - tile_kb0;  // blocks of the first set; the second has as many or one fewer
    const int kb0 = half ? tile_kb0 + steps : tile_kb0, kb1 = (half || SETS == 1) ? tile_kb1 : tile_kb0 + steps;

    bf16x8 qw[QS];
    {
      const bf16_t* qrow = a.q + (size_t)(q0 + (col_ok ? ti : 0)) * a.q_stride + head * HD;
#pragma unroll
      for (int i = 0; i < QS; ++i) {
        qw[i] = *reinterpret_cast<const bf16x8*>(qrow + i * 16 + h * 8);
        if (!col_ok) qw[i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    f32x16 o[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[ct][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;  // lsum: this lane's 16 keys of every block; its partner holds the other 16
    // The sums are rescaled when a block's maximum exceeds their reference by more than this (in the scores' units: a
    // factor 2^8 in the weights), not at every new maximum: in long rows of keys a new maximum somewhere among a tile's
    // tokens is frequent, a far larger one rare, and the rescaling is a pass over all sums.
    const float slack = 8.f / a.scale_log2;

    // This lane's pieces of a block: instruction wave * IPW + r of the keys and of the values.
    int k_key[IPW], k_off[IPW];  // the key of the block (0 .. 31) and the first channel of the piece
    int v_ch[IPW], v_key[IPW];   // the channel and the first key of the block (a multiple of 8)
#pragma unroll
    for (int r = 0; r < IPW; ++r) {
      const int ni = wave * IPW + r;
      const int rho = ni + NI * (lane / KP);                                            // LDS row of the keys
      k_key[r] = (rho & 16) + 8 * ((rho >> 2) & 1) + 4 * ((rho >> 3) & 1) + (rho & 3);  // the key that lives there
      k_off[r] = ((lane % KP) ^ (rho >> 4)) * 8;
      const int st = ni / CT, ch = 32 * (ni % CT) + lane / 2;
      v_ch[r] = ch;
      v_key[r] = 16 * st + 8 * ((lane & 1) ^ ((ch >> 4) & 1));
    }
    const int vlo = wlo & ~7, vhi = (whi - 1) & ~7;
    const size_t k_head = ((size_t)kvh * HD) << psh, kv_page = ((size_t)a.kv_heads * HD) << psh;  // elements
    const unsigned page_bytes = (unsigned)kv_page * 2;
    // Pages that divide a block: a block has 32 / PS of them, and which of them a lane's piece lies in, and where in it,
    // is the same in every block that lies wholly inside [wlo, whi).  Larger pages: a block lies in one.
    constexpr bool EVEN = PS <= 32;
    constexpr int PPB = EVEN ? 32 / PS : 1;  // pages per block
    int k_slot[IPW], v_slot[IPW], k_const[IPW], v_const[IPW];
#pragma unroll
    for (int r = 0; r < IPW; ++r) {
      k_slot[r] = EVEN ? k_key[r] >> psh : 0;
      v_slot[r] = EVEN ? v_key[r] >> psh : 0;
      k_const[r] = (int)k_head + (k_key[r] & pmask) * HD + k_off[r];
      v_const[r] = (int)k_head + (v_ch[r] << psh) + (v_key[r] & pmask);
    }
    auto inside = [&](int kb) { return EVEN && kb * 32 >= wlo && kb * 32 + 31 < whi; };
    // A block's page ids are the same for every lane, so they are read through the scalar unit (the constant address
    // space: this kernel does not write the table) and live in scalar registers; a lane picks its own.  Slots are kept
    // inside the held pages: a key outside [wlo, whi) is masked anyway, and so any block may be asked for.
    typedef const __attribute__((address_space(4))) int* scalar_ints;
    const scalar_ints stable = (scalar_ints)(unsigned long long)table;
    const int lo_slot = wlo >> psh, hi_slot = max((whi - 1) >> psh, lo_slot);  // (a tile without tokens sees no key: slot 0 of its row)
    auto page_ids = [&](int(&ids)[PPB], int kb) {
      const int first = (kb * 32) >> psh;
#pragma unroll
      for (int p = 0; p < PPB; ++p) ids[p] = stable[min(max(first + p, lo_slot), hi_slot)];
    };
    auto pick = [&](const auto(&per_page)[PPB], int slot) {  // per_page[slot], with per_page in scalar registers
      auto x = per_page[0];
#pragma unroll
      for (int p = 1; p < PPB; ++p) {
        x = slot == p ? per_page[p] : x;
        // (kept a chain of selects: rewritten as an array indexed by the lane's slot, the ids would move to scratch
        // memory, whose accesses count among the loads that the rounds' waits count)
        if (PPB > 2) asm volatile("" : "+v"(x));
      }
      return x;
    };
    typedef __attribute__((address_space(3))) void* lds_ptr;
    auto load_k = [&](const int(&ids)[PPB], int kb, int slot) {  // the keys of block kb into ring buffer `slot`
      const bool in = inside(kb);
#pragma unroll
      for (int r = 0; r < IPW; ++r) {
        const int id = pick(ids, k_slot[r]);
        const bf16_t* src;
        if (in) {
          src = a.k_cache + (size_t)id * kv_page + k_const[r];
        } else {
          const int key = min(max(kb * 32 + k_key[r], wlo), whi - 1);
          src = a.k_cache + (size_t)id * kv_page + k_head + (size_t)(key & pmask) * HD + k_off[r];
        }
        __builtin_amdgcn_global_load_lds(src, (lds_ptr)(kring + slot * K_BUF + (wave * IPW + r) * K_REGION), 16, 0, 0);
      }
    };
    auto load_v = [&](const int(&ids)[PPB], int kb, int slot) {
      const bool in = inside(kb);
#pragma unroll
      for (int r = 0; r < IPW; ++r) {
        const int id = pick(ids, v_slot[r]);
        const bf16_t* src;
        if (in) {
          src = a.v_cache + (size_t)id * kv_page + v_const[r];
        } else {
          const int key8 = min(max(kb * 32 + v_key[r], vlo), vhi);
          src = a.v_cache + (size_t)id * kv_page + k_head + ((size_t)v_ch[r] << psh) + (key8 & pmask);
        }
        __builtin_amdgcn_global_load_lds(src, (lds_ptr)(vring + slot * V_BUF + (wave * IPW + r) * 1024), 16, 0, 0);
      }
    };

    // Where this lane reads: its key row c at (c % NI, c / NI), the piece pair's half by bit 4 of the row; its channel
    // 32 ct + c of a plane, the half of its 32 bytes by bit 4 of the channel.  One address each, constant offsets.
    const int hs = (h ^ (c >> 4)) * 16;
    const int k_read = half * SET_BYTES + (c % NI) * K_REGION + (c / NI) * (KP * 16) + hs;
    const int v_read = half * SET_BYTES + RING * K_BUF + c * 32 + hs;
    // (the sum of a lane's part and a ring buffer's is formed once per round, the pieces lie at constant offsets from it)
    auto k_at = [&](int slot) {
      int at = k_read + slot * K_BUF;
      asm volatile("" : "+v"(at));
      return at;
    };
    auto v_at = [&](int slot) {
      int at = v_read + slot * V_BUF;
      asm volatile("" : "+v"(at));
      return at;
    };
    auto k_piece = [&](int at, int i) { return *reinterpret_cast<const bf16x8*>(smem + at + 32 * i); };
    auto v_piece = [&](int at, int t) { return *reinterpret_cast<const bf16x8*>(smem + at + (t / CT) * V_PLANE + (t % CT) * 1024); };  // t: key half major
    f32x16 s;  // the scores of the block whose turn is next: s[r] is key 16 (r / 8) + 8 h + r % 8 of token c
    auto scores = [&](int slot) {
      const int at = k_at(slot);
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
      for (int i = 0; i < QS; ++i) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_piece(at, i), qw[i], s, 0, 0, 0);
    };
    auto weigh = [&](int slot, const bf16x8(&pf)[2]) {
      const int at = v_at(slot);
#pragma unroll
      for (int t = 0; t < 2 * CT; ++t) o[t % CT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_piece(at, t), pf[t / CT], o[t % CT], 0, 0, 0);
    };

    // Before the first round: the keys of blocks 0, 1 and 2 and the values of blocks 0 and 1 are in their ring buffers, the
    // scores of block 0 are formed, and the page ids of blocks 3 and 2 are at hand for the keys and the values that
    // first round asks for.
    int ids_k[PPB], ids_v[PPB];
    {
      const int nb = kb1 - kb0;
      int i0[PPB], i1[PPB];
      page_ids(i0, kb0);
      page_ids(i1, kb0 + 1);
      page_ids(ids_v, kb0 + 2);
      page_ids(ids_k, kb0 + 3);
      if (nb > 0) {
        load_k(i0, kb0, 0);
        load_v(i0, kb0, 0);
      }
      if (nb > 1) {
        load_k(i1, kb0 + 1, 1);
        load_v(i1, kb0 + 1, 1);
      }
      if (nb > 2) load_k(ids_v, kb0 + 2, 2);
    }
    // (loads land in the order they were asked for: the first scores wait for the keys of block 0 only, the first round for the
    // values of block 0 and the keys of block 1; a range of fewer than three blocks waits for all it asked for)
    if (kb1 - kb0 > 2)
      NS_WAIT_LOADS(4 * IPW);
    else
      NS_WAIT_LOADS(0);
    __builtin_amdgcn_s_barrier();
    if (head_ok && kb0 < kb1) scores(0);
    if (kb1 - kb0 > 2) NS_WAIT_LOADS(2 * IPW);
    __builtin_amdgcn_s_barrier();  // (the scores' LDS reads are done: a matrix instruction has taken each of them)

    // What round `it` asks for: the keys of block it + 3 over those of block it, whose scores are formed, and the values
    // of block it + 2 over those of block it - 1.  It returns the number of load instructions.
    auto ask = [&](int it, auto near_tag) -> int {
      constexpr bool NEAR = decltype(near_tag)::value;
      const int kb = kb0 + it;
      int asked = 0;
      if (kb + 3 < kb1) {
        const int slot = it % RING;
        if (NEAR && inside(kb + 3)) {  // a pool within 4 GiB: offsets of 32 bits, a page's formed by the scalar unit
          unsigned pages[PPB];
#pragma unroll
          for (int p = 0; p < PPB; ++p) pages[p] = (unsigned)ids_k[p] * page_bytes;
#pragma unroll
          for (int r = 0; r < IPW; ++r) {
            const char* src = reinterpret_cast<const char*>(a.k_cache) + (pick(pages, k_slot[r]) + (unsigned)k_const[r] * 2);
            __builtin_amdgcn_global_load_lds(src, (lds_ptr)(kring + slot * K_BUF + (wave * IPW + r) * K_REGION), 16, 0, 0);
          }
        } else {
          load_k(ids_k, kb + 3, slot);
        }
        asked += IPW;
      }
      if (kb + 2 < kb1) {
        const int slot = (it + 2) % RING;
        if (NEAR && inside(kb + 2)) {
          unsigned pages[PPB];
#pragma unroll
          for (int p = 0; p < PPB; ++p) pages[p] = (unsigned)ids_v[p] * page_bytes;
#pragma unroll
          for (int r = 0; r < IPW; ++r) {
            const char* src = reinterpret_cast<const char*>(a.v_cache) + (pick(pages, v_slot[r]) + (unsigned)v_const[r] * 2);
            __builtin_amdgcn_global_load_lds(src, (lds_ptr)(vring + slot * V_BUF + (wave * IPW + r) * 1024), 16, 0, 0);
          }
        } else {
          load_v(ids_v, kb + 2, slot);
        }
        asked += IPW;
      }
      return asked;
    };
    // Every round ends the same way: the loads that the round before asked for have landed (this round's may still be
    // on their way), and all waves have read what this round reads.
    auto round_end = [&](int asked) {
      if (asked == 2 * IPW)
        NS_WAIT_LOADS(2 * IPW);
      else if (asked == IPW)
        NS_WAIT_LOADS(IPW);
      else
        NS_WAIT_LOADS(0);
      __builtin_amdgcn_s_barrier();
    };
    // One round of the general form.  Both sets pass every barrier; the second may have no block in the last round.
    auto round = [&](int it, auto full_tag) {
      constexpr bool FULL = decltype(full_tag)::value;
      const int kb = kb0 + it;
      const int ks = (it + 1) % RING, vs = it % RING;  // where the keys of block it + 1 and the values of block it lie
      int ids_next[PPB];
      page_ids(ids_next, kb + 4);
      const int asked = ask(it, std::false_type{});
      if (head_ok && kb < kb1) {
        const int key_base = kb * 32;
        f32x16 cur = s;
        if (kb + 1 < kb1) scores(ks);
        if (!FULL) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = key_base + 16 * (r >> 3) + 8 * h + (r & 7);
            cur[r] = (key >= lo && key <= pos) ? cur[r] : -INFINITY;
          }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, cur[r]);
        mx = max_with_other_half(mx);
        // m is what the sums refer to: a maximum of the raw scores so far (the scale is positive), followed only when the
        // maximum has moved far, since weights up to 2^8 lose nothing; p = 2^((s - m) scale log2 e)
        const float m_new = mx > m + slack ? mx : m;
        const float m_safe = (!FULL && m_new == -INFINITY) ? 0.f : m_new;  // (a full block's maximum is a score)
        const bool moved = m_new != m;
        const float shift = -m_safe * a.scale_log2;
        bf16x8 pf[2];
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fast_exp2(fmaf(cur[r], a.scale_log2, shift));
          psum += p;
          pf[r >> 3][r & 7] = (bf16_t)p;
        }
        if (__any(moved)) {  // the maximum settles early in long rows; rescaling is skipped from then on
          const float alpha = fast_exp2((m - m_safe) * a.scale_log2);
          lsum *= alpha;
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[ct][r] *= alpha;
        }
        m = m_new;
        lsum += psum;
        weigh(vs, pf);
      }
#pragma unroll
      for (int p = 0; p < PPB; ++p) {
        ids_v[p] = ids_k[p];
        ids_k[p] = ids_next[p];
      }
      round_end(asked);
    };
    // A round whose block is seen wholly by every token and is not the range's last, in a wave that has a head: straight
    // code in two stages,
    //   A  the scores of block it + 1 (matrix instructions)  beside  the soft-max weights of block it (vector instructions)
    //   B  the weighted values of block it, and beside the first of them the other half of the weights
    // (the rescaling of the sums stands between the stages and runs only when a maximum moved).
    auto steady = [&](int it, auto near_tag, auto guarded_tag) {
      constexpr bool NEAR = decltype(near_tag)::value;
      constexpr bool GUARDED = decltype(guarded_tag)::value;  // near the range's end, where not every load is asked for
      const int kb = kb0 + it;
      const int ks = (it + 1) % RING, vs = it % RING;
      int ids_next[PPB];  // (asked for at the round's end: an LDS read's wait would wait for them too)
      int asked = 2 * IPW;
      if (GUARDED) {
        asked = ask(it, near_tag);
      } else if (NEAR) {  // a pool within 4 GiB: offsets of 32 bits, a page's formed by the scalar unit
        unsigned k_pages[PPB], v_pages[PPB];
#pragma unroll
        for (int p = 0; p < PPB; ++p) {
          k_pages[p] = (unsigned)ids_k[p] * page_bytes;
          v_pages[p] = (unsigned)ids_v[p] * page_bytes;
        }
#pragma unroll
        for (int r = 0; r < IPW; ++r) {
          const char* ksrc = reinterpret_cast<const char*>(a.k_cache) + (pick(k_pages, k_slot[r]) + (unsigned)k_const[r] * 2);
          const char* vsrc = reinterpret_cast<const char*>(a.v_cache) + (pick(v_pages, v_slot[r]) + (unsigned)v_const[r] * 2);
          __builtin_amdgcn_global_load_lds(ksrc, (lds_ptr)(kring + vs * K_BUF + (wave * IPW + r) * K_REGION), 16, 0, 0);
          __builtin_amdgcn_global_load_lds(vsrc, (lds_ptr)(vring + ((it + 2) % RING) * V_BUF + (wave * IPW + r) * 1024), 16, 0, 0);
        }
      } else {
#pragma unroll
        for (int r = 0; r < IPW; ++r) {
          const bf16_t* ksrc = a.k_cache + (size_t)pick(ids_k, k_slot[r]) * kv_page + k_const[r];
          const bf16_t* vsrc = a.v_cache + (size_t)pick(ids_v, v_slot[r]) * kv_page + v_const[r];
          __builtin_amdgcn_global_load_lds(ksrc, (lds_ptr)(kring + vs * K_BUF + (wave * IPW + r) * K_REGION), 16, 0, 0);
          __builtin_amdgcn_global_load_lds(vsrc, (lds_ptr)(vring + ((it + 2) % RING) * V_BUF + (wave * IPW + r) * 1024), 16, 0, 0);
        }
      }
      // The order of issue is written out, a chunk per matrix instruction, and fixed by a scheduling barrier after each:
      // the LDS read of the operand two instructions ahead, the matrix instruction, a piece of the vector arithmetic.
      // ---- A
      const f32x16 cur = s;
      const int kat = k_at(ks), vat = v_at(vs);
      // Operands come from LDS in bursts of half a stage's, asked for right after the first matrix instruction of the
      // burst before has waited for its own: a wait for LDS waits for every read on its way, so a burst is asked for
      // where no other is outstanding, and has the time of the burst before it to arrive.
      constexpr int BS = QS / 2;
      static_assert(2 * CT == QS && BS >= 1, "a stage has as many matrix instructions for the values as for the scores");
      bf16x8 ka[QS], va[2 * CT];
#pragma unroll
      for (int u = 0; u < BS; ++u) ka[u] = k_piece(kat, u);
      float mx = -INFINITY, m_new = m, shift = 0.f, psum = 0.f, pv[16];
      bool moved = false;
      bf16x2 ph[8];
      auto weight = [&](int r) {  // the weight of score r; a pair is rounded together
        pv[r] = fast_exp2(fmaf(cur[r], a.scale_log2, shift));
        psum = r == 0 ? pv[r] : psum + pv[r];
        if (r & 1) {
          ph[r >> 1] = __builtin_convertvector(f32x2{pv[r - 1], pv[r]}, bf16x2);
          asm volatile("" : "+v"(ph[r >> 1]), "+v"(psum));  // formed here, beside the matrix instruction, not where it is used
        } else {
          asm volatile("" : "+v"(pv[r]));
        }
      };
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, cur[r]);
      asm volatile("" : "+v"(mx));
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.f;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < QS; ++i) {
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[i], qw[i], s, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (i % BS == 0) {
#pragma unroll
          for (int u = 0; u < BS; ++u) {
            if (i + BS < QS)
              ka[i + BS + u] = k_piece(kat, i + BS + u);
            else
              va[u] = v_piece(vat, u);
          }
        }
        if (i == 0) {
          mx = max_with_other_half(mx);
          m_new = mx > m + slack ? mx : m;
          moved = __any(m_new != m);
          shift = -m_new * a.scale_log2;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e * QS / 8 == i) weight(e);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (moved) {
        const float alpha = fast_exp2((m - m_new) * a.scale_log2);
        lsum *= alpha;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[ct][r] *= alpha;
      }
      m = m_new;
      // ---- B: the first half of the keys in every tile of channels, then the second, whose weights are formed meanwhile
      bf16x8 pf[2];
      pf[0] = __builtin_shufflevector(__builtin_shufflevector(ph[0], ph[1], 0, 1, 2, 3), __builtin_shufflevector(ph[2], ph[3], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int t = 0; t < 2 * CT; ++t) {
        if (t == CT)
          pf[1] = __builtin_shufflevector(__builtin_shufflevector(ph[4], ph[5], 0, 1, 2, 3), __builtin_shufflevector(ph[6], ph[7], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
        o[t % CT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[t], pf[t / CT], o[t % CT], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (t % BS == 0 && t + BS < 2 * CT) {
#pragma unroll
          for (int u = 0; u < BS; ++u) va[t + BS + u] = v_piece(vat, t + BS + u);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e * CT / 8 == t) weight(8 + e);
        if (t == 2 * CT - 1) page_ids(ids_next, kb + 4);
        __builtin_amdgcn_sched_barrier(0);
      }
      lsum += psum;
#pragma unroll
      for (int p = 0; p < PPB; ++p) {
        ids_v[p] = ids_k[p];
        ids_k[p] = ids_next[p];
      }
      if (GUARDED) {
        round_end(asked);
      } else {
        NS_WAIT_LOADS(2 * IPW);
        __builtin_amdgcn_s_barrier();
      }
    };

    // The first blocks of this set's range that every token of the tile sees wholly run the forms without masks.  Both
    // sets pass a barrier in every round, whichever form a round takes.
    const int seen_whole = a.window > 0 ? 0 : min(max((full_hi + 1) / 32 - kb0, 0), max(kb1 - kb0, 0));
    // (steady: every block that is asked for, up to block it + 4's ids, lies wholly inside the tile's keys and the range)
    const int n_fast = head_ok ? min(seen_whole, kb1 - kb0 - 1) : 0;
    const int n_steady = EVEN ? max(min(n_fast, kb1 - kb0 - 4), 0) : 0;
    int it = 0;
    if (a.near) {
      for (; it < n_steady; ++it) steady(it, std::true_type{}, std::false_type{});
      for (; it < n_fast; ++it) steady(it, std::true_type{}, std::true_type{});
    } else {
      for (; it < n_steady; ++it) steady(it, std::false_type{}, std::false_type{});
      for (; it < n_fast; ++it) steady(it, std::false_type{}, std::true_type{});
    }
    for (; it < seen_whole; ++it) round(it, std::true_type{});
    for (; it < steps; ++it) round(it, std::false_type{});

    // a token's total: this lane's keys and its partner's
    lsum += __shfl_xor(lsum, 32, 64);
    // The second set hands its sums to the first, lane by lane (both hold the same tokens and channels):
    // o = o_0 2^((m_0 - m*) scale) + o_1 2^((m_1 - m*) scale), likewise the totals, m* = max(m_0, m_1).
    if (SETS == 2) __syncthreads();  // the ring is read no more: the hand-over lies over it
    float* join = reinterpret_cast<float*>(smem) + tid * JOIN;
    if (SETS == 2 && half) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int r = 0; r < 16; r += 4) *reinterpret_cast<f32x4*>(join + ct * 16 + r) = f32x4{o[ct][r], o[ct][r + 1], o[ct][r + 2], o[ct][r + 3]};
      join[CT * 16] = m;
      join[CT * 16 + 1] = lsum;
    }
    if (SETS == 2) __syncthreads();
    if (half) return;
    if (SETS == 2) {
      const float m1 = join[CT * 16], l1 = join[CT * 16 + 1];
      const float mstar = fmaxf(m, m1);
      const float msafe = mstar == -INFINITY ? 0.f : mstar;
      const float w0 = fast_exp2((m - msafe) * a.scale_log2), w1 = fast_exp2((m1 - msafe) * a.scale_log2);
      lsum = lsum * w0 + l1 * w1;
      m = mstar;  // what the sums now refer to: a range's maximum goes out with them
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int r = 0; r < 16; r += 4) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(join + ct * 16 + r);
#pragma unroll
          for (int j = 0; j < 4; ++j) o[ct][r + j] = o[ct][r + j] * w0 + v[j] * w1;
        }
    }

    if (!col_ok) return;
    // o[ct][4 bb + j] is channel 32 ct + 8 bb + 4 h + j of token c
    if (a.splits == 1) {
      const size_t col = (size_t)(q0 + t0 + c) * a.heads + head;
      const float inv = 1.f / lsum;
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          bf16x4 r = {(bf16_t)(o[ct][4 * bb] * inv), (bf16_t)(o[ct][4 * bb + 1] * inv), (bf16_t)(o[ct][4 * bb + 2] * inv),
                      (bf16_t)(o[ct][4 * bb + 3] * inv)};
          *reinterpret_cast<bf16x4*>(a.out + col * HD + 32 * ct + 8 * bb + 4 * h) = r;
        }
    } else {  // as the ranges of a decode tile: unnormalised sums, maximum in the exponent's units, total
      const size_t pcol = ((size_t)tile * 32 + c) * a.heads + head;
      float* po = a.part_o + (pcol * a.splits + split) * HD;
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb)
          *reinterpret_cast<f32x4*>(po + 32 * ct + 8 * bb + 4 * h) = f32x4{o[ct][4 * bb], o[ct][4 * bb + 1], o[ct][4 * bb + 2], o[ct][4 * bb + 3]};
      if (h == 0) {
        a.part_ml[(pcol * a.splits + split) * 2] = m * a.scale_log2;
        a.part_ml[(pcol * a.splits + split) * 2 + 1] = lsum;
      }
    }
  }
}
