// fp16 3x3 stride-1 pad-1 convolution + BN/residual/activation for gfx950: the stream form of the LDS-patch
// kernel (conv3x3_patch.hip keeps every other case: fp32, stride 2, odd channel counts, wide rows, more than 256
// channels, and launches too small to fill the CUs, where its shorter prologue wins).
// Replaces what ModernTile.cpp:184-199 + ModernVec.cpp:54-62 emit for linalg.conv_2d_nchw_fchw
// (tests/Nets/Res18.mlir:157 ...) together with the BN / add / ReLU generics behind it (:127-142, :193-203).
//
// What is different from conv3x3_patch.hip, and why:
//  * A workgroup is persistent: it owns one block of filters and walks a list of pixel tiles.  The
//    haloed input patch of the NEXT (tile, channel slab) is requested before the taps of the current one
//    and goes from global memory straight into the other of two LDS buffers (buffer_load ... lds, 16 bytes
//    per lane: no staging registers, no LDS store instructions), so a slab change costs one barrier and no
//    wait, and the weight stream (fragment-major, straight from global memory into registers, nine K steps
//    ahead) never stops at a tile boundary.
//  * A wave owns 128 pixel slots x 32 filters (four 32x32x16 MFMAs per K step share ONE weight fragment):
//    per MFMA the vector-memory path carries 256 bytes of weights instead of 512, and LDS (256 B/clk
//    on this chip) carries the pixels.  The 64 B/clk vector-memory path was what a 2x2 blocking saturated.
//  * All addressing is arithmetic on the block and lane ids with host-computed reciprocals: no tables in
//    memory, no dependent loads before the first patch request, no divisions.
//  * Rows of all images are stacked into one column of "virtual rows"; a tile is TH consecutive virtual
//    rows.  Either every image takes a whole number of tiles (aligned form), or the images are one zero
//    row apart and tiles run across image borders (gap form: that shared row is the halo of both images);
//    14x14 and 7x7 images fill 126 of 128 slots that way instead of 98.
//  * Patch cells (the 64 channels of one pixel, 128 bytes) are 144 bytes apart in LDS, which keeps the 16-byte
//    reads of 16 neighbouring cells off each other's banks (64 banks of 4 bytes: a read is conflict-free when its
//    16-byte units differ mod 16 within every 16 lanes, and 9 is odd).  Consecutive pixel slots wrap from the
//    end of one patch row to the start of the next, so the pitch of a patch row is chosen to continue that
//    sequence: row pitch = 9 W units (mod 16), which for W a multiple of seven is one 16-byte unit more than the
//    row's segments.  Slots past the last pixel of a tile read the cell of the slot 16, 32 .. before them (same
//    bank group, never a conflict).  Measured with a micro-benchmark of the read alone: 28 and 14 pixel rows at
//    the plain segment pitch cost 1.6x and 2.1x the cycles of a conflict-free read, at this pitch 1.0x.
//    A load instruction fills a row segment of seven cells: 63 lanes x 16 bytes = 7 x 144 (lane 63 writes what
//    lane 0 of the next segment overwrites, or the spare unit at the end of the row).
//    Which pixel a lane fetches is worked out once per tile, one segment per lane, and dealt to the nine
//    load instructions of a wave with ds_bpermute; a lane whose cell is padding, halo outside the image or
//    past the tile asks for an offset beyond the buffer and gets zeros.  Every wave issues all nine loads
//    in every stage, so the compiler's count of outstanding loads is exact and the weight ring is never
//    over-waited.
//  * Inside a stage each MFMA is followed by its share of the other work (next K step's LDS reads, a weight
//    refill, a piece of the next patch) and pinned there, so the matrix pipe is issued to at a steady rate.
//    The two workgroups of a CU take turns at the higher wave priority, tile by tile.
//  * The filters of a wave are stored permuted (row 8q+4h+e of the MFMA holds filter 16h+4q+e), so a
//    lane ends up with 16 consecutive output channels of a pixel: results go from the accumulators to
//    memory with two 16-byte stores, without a transposing pass through LDS.  K groups (the waves that
//    split the channel slab) exchange half of their partial sums through LDS once per tile.
#include <algorithm>

#include "arena_plan.hpp"
#include "mfma_tile.hpp"
#include "runtime.hpp"

namespace nncv_hip {

using namespace mt;

namespace {

constexpr int kSlots = 128;                       // pixel slots per pixel group of a workgroup tile
constexpr int kPitchS = 144;                      // LDS bytes per patch cell: 128 payload + 16 pad (conflict-free 16-byte reads)
constexpr int kSegCells = 7;                      // patch cells one load instruction fills: 63 lanes x 16 bytes = 7 x 144
constexpr int kSegB = kSegCells * kPitchS;        // 1008 bytes
constexpr int kLoadsPerWave = 9;                  // patch load instructions per wave and stage, always all issued
// row segments per patch buffer and its bytes (the segments, the 16 bytes the last lane of the last one writes and
// the units that bring the row pitch to 9 W mod 16) for a workgroup of nw waves: 39424 bytes for four waves, 75712 for eight
constexpr int seg_cap(int nw) { return nw * kLoadsPerWave; }
constexpr int kRowPadB = 3072;
constexpr int patch_bytes(int nw) { return seg_cap(nw) * kSegB + 64 + kRowPadB; }
constexpr unsigned kOOBs = 0x80000000u;           // buffer offsets at or above this are out of range
constexpr int kRing = 9;                          // weight fragments in flight per wave (K steps ahead)
constexpr int kXcds = 8;

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// 16 bytes per lane from global memory straight into LDS: lane l to lds + 16 l.  A function of its own: with the builtin
// called from the kernel template itself, the host pass of hipcc 7.2 can emit no launch stub for the kernel (and no
// message), depending on the code around the call.
__device__ __forceinline__ void load_to_lds16(__amdgpu_buffer_rsrc_t rs, unsigned char* lds, unsigned voffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)lds, 16, voffset, 0, 0, 0);
}

// s_waitcnt immediate that waits for all but the n youngest vector-memory operations and for nothing else
constexpr int vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0070 | 0x0f00; }

struct StreamArgs {
  // ---- what the first requests need.  The kernel takes these 14 dwords as plain leading arguments: those arrive
  //      preloaded in SGPRs at wave launch (a struct passed by value does not: its fields come by scalar loads, three
  //      of them in a row here before the first weight request could go out), the rest follows as a struct ----
  const void* in;         // NHWC [N][H][W][pix]
  const void* wf;         // launch_weight_frag32 order
  unsigned G, div, mdiv;  // workgroup -> (filter block, first tile): see launch_conv3x3_stream
  unsigned mS32;          // ceil(2^32 / S)
  unsigned n_tiles;
  unsigned tstep_nslab_flags;  // tile step | channel slabs << 16 | by_filter << 24 | aligned << 25 | top << 26
  unsigned N_TH;               // N | TH << 24
  unsigned geom;               // H | W << 8 | S << 16 | NSEG << 24
  unsigned pixB;               // bytes between input pixels
  unsigned rowx_rnseg;         // bytes a patch row is longer than its segments | ceil(2^16 / NSEG) << 16 (0 when NSEG is 1)
  // ---- the end of a tile needs these ----
  struct Tail {
    void* out;              // NHWC [N][H][W][ldo]
    const float* scale;     // [F] or null
    const float* shift;     // [F] or null
    const void* residual;   // like out, or null
    unsigned out_bytes, mW16;  // mW16 = ceil(2^16 / W)
    int F, act, ldo;
  } t;
};
// Input and weights are addressed through descriptors of 2^31 bytes: every offset the kernel forms for a cell or a
// fragment that exists lies inside its tensor (the host checks the sizes), and what must read as zero carries kOOBs.
constexpr unsigned kWholeRange = 0x80000000u;

// Geometry: rows of all images are stacked into virtual rows, image n's row y being v = n*S + top + y; tile t
// covers virtual rows [top + t*TH, +TH) and W columns.  The patch of a tile is its TH + 2 rows of W + 2 cells,
// each row padded to NSEG segments of 7 cells in LDS.
//
// PG x WF x WK waves: PG pixel groups of up to four 32-slot rows (a tile is up to 128*PG pixel slots), WF filter
// groups of 32 (the workgroup's filter block is 32*WF filters), WK K groups.  Four waves: two workgroups per CU;
// eight waves: one, whose waves w and w + 4 share a SIMD -- one of each pixel group, so that a tile of seven
// rows (four + three) loads all SIMDs alike.
//
// RES: a layer of one channel slab (64 channels) has kSteps weight fragments per wave in all; they stay in registers for
// the life of the workgroup instead of passing through the ring again for every tile.
template <int PG, int WF, int WK, bool ACT, bool RES = false>
__global__ __launch_bounds__(64 * PG * WF * WK) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv3x3_f16_stream_kernel(
    const void* in_p, const void* wf_p, unsigned G_p, unsigned div_p, unsigned mdiv_p, unsigned mS32_p, unsigned n_tiles_p,
    unsigned flags_p, unsigned N_TH_p, unsigned geom_p, unsigned pixB_p, unsigned rowx_rnseg_p, const StreamArgs::Tail tail) {
  StreamArgs a;
  a.in = in_p; a.wf = wf_p; a.G = G_p; a.div = div_p; a.mdiv = mdiv_p; a.mS32 = mS32_p; a.n_tiles = n_tiles_p;
  a.tstep_nslab_flags = flags_p; a.N_TH = N_TH_p; a.geom = geom_p; a.pixB = pixB_p; a.rowx_rnseg = rowx_rnseg_p;
  a.t = tail;
  static_assert(WF * WK == 4 && (PG == 1 || PG == 2), "four or eight waves");
  constexpr int NW = PG * WF * WK;
  constexpr int kPatchB = patch_bytes(NW);
  constexpr int KPG = 4 / WK;        // 32-byte K sub-steps of a tap per K group
  constexpr int kSteps = 9 * KPG;    // K steps per (tile, slab) stage and wave
  constexpr int NOWN = 4 / WK;       // pixel groups of 32 slots a wave finishes in the epilogue
  constexpr int BF = 32 * WF;        // filters per workgroup
  static_assert(kSteps % kRing == 0 || kRing % kSteps == 0, "the weight ring must tile a stage");
  constexpr int kW = RES ? kSteps : kRing;  // weight fragments a wave holds
  constexpr int kPieceSteps = KPG >= 2 ? 9 : 5;  // K steps of a stage that carry the next patch's load instructions
  static_assert(kPieceSteps + 1 < kSteps, "the last piece is loaded in step kPieceSteps, the residual rows one step later");
  // weight refills younger than the last patch piece (loaded in step kPieceSteps, ahead of that step's refill) at the end of
  // a stage: what the wait for the patch may leave in flight
  // (resident weights: no refills; the residual rows' loads of the stage are what follows the last piece)
  constexpr int kYoung = RES ? 2 * NOWN : (kSteps - kPieceSteps < kRing ? kSteps - kPieceSteps : kRing);
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pg = wave / 4, wf = (wave % 4) % WF, wk = (wave % 4) / WF;
  const int lrow = lane & 31, lchunk = lane >> 5;

  const int tstep = (int)(a.tstep_nslab_flags & 0xffffu), nslab = RES ? 1 : (int)((a.tstep_nslab_flags >> 16) & 0xffu);
  const bool by_filter = (a.tstep_nslab_flags >> 24) & 1u, aligned = (a.tstep_nslab_flags >> 25) & 1u;
  const unsigned top = (a.tstep_nslab_flags >> 26) & 1u;
  const unsigned N = a.N_TH & 0xffffffu, TH = a.N_TH >> 24;
  const unsigned H = a.geom & 0xffu, W = (a.geom >> 8) & 0xffu, S = (a.geom >> 16) & 0xffu, NSEG = a.geom >> 24;
  const int XB = (int)(a.rowx_rnseg & 0xffffu);  // spare bytes behind the segments of a patch row
  const int RPB = (int)NSEG * kSegB + XB;        // LDS bytes from one patch row to the next
  const unsigned rnseg = a.rowx_rnseg >> 16;
  // 32-slot rows of the tile this wave's pixel group holds: four, or what is left of the tile's
  const int trows = (int)((TH * W + 31u) >> 5);
  const int nrows = PG == 1 ? 4 : (trows - 4 * pg < 4 ? (trows - 4 * pg < 0 ? 0 : trows - 4 * pg) : 4);

  // ---- workgroup -> filter block and tile list.  Hardware deals workgroups to the 8 XCDs round-robin by
  //      linear id; `logical` makes an XCD's workgroups neighbours in the (filter block, tile) order ----
  const unsigned bid = blockIdx.x;
  const unsigned logical = (bid & (kXcds - 1)) * ((a.G + kXcds - 1) / kXcds) + (bid / kXcds);
  if (logical >= a.G) return;
  const unsigned qd = a.div == 1 ? logical : __umulhi(logical, a.mdiv);
  const unsigned rd = logical - qd * a.div;
  const int fb = (int)(by_filter ? qd : rd);
  int tile = (int)(by_filter ? rd : qd);
  const int tend = (int)a.n_tiles;
  if (tile >= tend) return;

  const __amdgpu_buffer_rsrc_t rs_wf = make_rsrc(a.wf, kWholeRange);

  // ---- weights: fragment (filter group g, iteration it = slab*9 + tap, sub-step kk) is the kilobyte at
  //      ((g*niter + it)*4 + kk)*1024; a wave streams its KPG sub-steps of every iteration ----
  const int niter = nslab * 9;
  const int wbase = ((fb * WF + wf) * niter * 4 + wk * KPG) * 1024;
  const unsigned wlane = lane * 16;
  const int wwrap = niter * 4096;
  u32x4 wring[kW];
  // step L (counted over the whole stream of the wave, KPG per iteration) lives at wbase + (L / KPG) * 4096 + (L % KPG) * 1024
  auto wload_at = [&](int soff) { return __builtin_amdgcn_raw_buffer_load_b128(rs_wf, wlane, wbase + soff, 0); };
  auto ring_fill = [&](auto q_c) {
    constexpr int q = decltype(q_c)::value;
    int it = q / KPG;
    if (it >= niter) it -= niter;  // a one-slab layer wraps inside the first ring fill
    wring[q] = wload_at(it * 4096 + (q % KPG) * 1024);
  };
  // the first fragments go out ahead of the patch request (they gate the first MFMA as much as the patch
  // does); the rest follow it, so that the patch is not queued behind 72 KB of weights per CU
  ring_fill(std::integral_constant<int, 0>());
  ring_fill(std::integral_constant<int, 1>());
  ring_fill(std::integral_constant<int, 2>());

  // ---- patch loader.  One load instruction (buffer_load ... lds: global memory straight into LDS, lane l
  //      to the instruction's LDS base + 16*l) fills one row segment: 63 lanes = chunk l % 9 of cell l / 9
  //      of the segment's 7 cells, chunk 8 being the pad of the 144-byte cell pitch; lane 63 is the first
  //      unit of the NEXT segment, which it loads like that segment's lane 0 does (the same bytes to the same
  //      place).  The patch buffer is kSegCap segments in row-major order, wave w loading segments 9w .. 9w+8:
  //      63 cells, whose tensor offsets (or an out-of-range offset for cells outside the image: the load then
  //      returns zeros) one lane each computes once per tile; an instruction's lanes fetch their cell's
  //      offset from there with a lane permute.  Every wave issues all nine instructions in every stage:
  //      a fixed count, so the compiler's wait for a weight fragment older than a patch request never
  //      includes the request.  The pieces are spread over the first K steps of a stage, between its
  //      MFMAs: outside the tap loop an instruction costs its wave about eight idle cycles. ----
  const unsigned lcell = ((unsigned)lane * 57u) >> 9, lch = (unsigned)lane - lcell * 9u;  // lane / 9, lane % 9
  const unsigned lchoff = lch == 8u ? kOOBs : lch * 16u;
  const int perm0 = (int)lcell * 4;  // permute address of this lane's cell in the wave's first segment
  // the cell this lane computes offsets for: number lane of the wave's 63 (+ the first of the next wave's)
  const unsigned cseg = (unsigned)wave * kLoadsPerWave + (((unsigned)lane * 37u) >> 8);  // its segment: lane / 7
  const unsigned crow = NSEG == 1 ? cseg : (cseg * rnseg) >> 16;                           // its patch row: cseg / NSEG
  const unsigned ccol = (cseg - crow * NSEG) * kSegCells + ((unsigned)lane - (((unsigned)lane * 37u) >> 8) * 7u) - 1u;  // image column
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, kWholeRange);
  unsigned celloff = kOOBs;  // tensor offset of that cell for the tile being loaded
  unsigned pc_lchslab = 0;   // lchoff + the channel slab's byte offset in a pixel
  int pc_dst = 0;            // LDS offset of this wave's first segment in the buffer being filled
  auto patch_tile = [&](int t, bool live) {
    const unsigned v0 = top + (unsigned)t * TH;
    const unsigned nt = __umulhi(v0, a.mS32);
    // patch row crow is virtual row v0 - 1 + crow; counted one image further down so that the row above the
    // first image divides like the others (its image is then -1 and fails n < N)
    const unsigned vS = v0 - 1u + crow + S;
    const unsigned nS = __umulhi(vS, a.mS32);
    const unsigned n = nS - 1u, y = vS - nS * S - top;
    const unsigned bad = (unsigned)(y >= H) | (unsigned)(n >= N) | (unsigned)(ccol >= W) | (unsigned)(crow >= TH + 2u) |
                         (unsigned)(aligned & (n != nt)) | (unsigned)!live;
    // a cell that is not there gets exactly kOOBs, not its (meaningless) offset with the flag set: the pad lane of such a
    // cell adds a second kOOBs, the flags cancel, and what is left must be an offset inside the tensor (its first bytes,
    // into a pad nobody reads) -- the descriptor spans 2^31 bytes and would not stop anything else
    celloff = bad ? kOOBs : ((n * H + y) * W + ccol) * a.pixB;
  };
  auto patch_begin = [&](int slab, int dstbuf) {
    pc_lchslab = lchoff + (unsigned)slab * 128u;
    pc_dst = dstbuf + wave * (kLoadsPerWave * kSegB);
  };
  // segment 9 * wave + pp starts its row's spare bytes times its row further down than in a row of segments alone
  int segx[kLoadsPerWave];
#pragma unroll
  for (int pp = 0; pp < kLoadsPerWave; ++pp) {
    const unsigned sg = (unsigned)wave * kLoadsPerWave + (unsigned)pp;
    segx[pp] = pp * kSegB + (int)(NSEG == 1 ? sg : (sg * rnseg) >> 16) * XB;
  }
  // A piece's permute goes out a whole K step (five MFMAs) ahead of its load: LDS answers in order, so a load that
  // follows its permute by one MFMA waits for every LDS read in flight, the next step's pixel operands included.
  constexpr int kVo = 2 * ((kLoadsPerWave + kPieceSteps - 1) / kPieceSteps);  // permute results in flight
  unsigned pc_vo[kVo];
  auto patch_piece_perm = [&](auto p_c) {  // the lanes' cell offsets for piece p
    constexpr int pp = decltype(p_c)::value;
    pc_vo[pp % kVo] = (unsigned)__builtin_amdgcn_ds_bpermute(perm0 + 28 * pp, (int)celloff);
  };
  auto patch_piece_load = [&](auto p_c) {
    constexpr int pp = decltype(p_c)::value;
    // out of range stays out of range under this sum, except for the pad chunk of a cell that is itself out of
    // range (the two flags cancel): that unit then loads the tensor's first bytes into a pad nobody reads
    load_to_lds16(rs_in, smem + pc_dst + segx[pp], pc_vo[pp % kVo] + pc_lchslab);
  };
  // the first patch of a workgroup: nothing to hide the permutes' latency under, so all nine go out before the loads
  auto patch_all = [&]() {
    unsigned pv[kLoadsPerWave];
#pragma unroll
    for (int pp = 0; pp < kLoadsPerWave; ++pp) pv[pp] = (unsigned)__builtin_amdgcn_ds_bpermute(perm0 + 28 * pp, (int)celloff);
#pragma unroll
    for (int pp = 0; pp < kLoadsPerWave; ++pp)
      load_to_lds16(rs_in, smem + pc_dst + segx[pp], pv[pp] + pc_lchslab);
  };

  patch_tile(tile, true);
  patch_begin(0, 0);
  patch_all();
  __builtin_amdgcn_sched_barrier(0);
  auto ring_rest = [&](auto self, auto q_c) -> void {
    constexpr int q = decltype(q_c)::value;
    if constexpr (q < kW) {
      ring_fill(q_c);
      self(self, std::integral_constant<int, q + 1>());
    }
  };
  ring_rest(ring_rest, std::integral_constant<int, 3>());
  __builtin_amdgcn_sched_barrier(0);

  // ---- everything below needs the rest of the arguments ----
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(a.t.out, a.t.out_bytes);
  const __amdgpu_buffer_rsrc_t rs_res = make_rsrc(a.t.residual ? a.t.residual : a.t.out, a.t.residual ? a.t.out_bytes : 0u);

  // Scale and shift of the block's filters wait in LDS behind the patch buffers (32 registers less across
  // the taps).  They are requested here and written at the end of the first stage: writing them now would
  // wait for the youngest requests, i.e. for everything.
  const int sse = tid & (BF / 2 - 1);
  const bool ss_shift = sse >= BF / 4;
  floatx4 vsc, vsh;
  {
    const unsigned off = (unsigned)(fb * BF + 4 * (ss_shift ? sse - BF / 4 : sse)) * 4u;
    // a missing vector is a buffer of no bytes: the load returns zeros and the select later fills in 1 / 0
    const __amdgpu_buffer_rsrc_t rs_sc = make_rsrc(a.t.scale ? a.t.scale : a.in, a.t.scale ? (unsigned)a.t.F * 4u : 0u);
    const __amdgpu_buffer_rsrc_t rs_sh = make_rsrc(a.t.shift ? a.t.shift : a.in, a.t.shift ? (unsigned)a.t.F * 4u : 0u);
    vsc = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rs_sc, off, 0, 0));
    vsh = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rs_sh, off, 0, 0));
  }
  bool ss_pending = true;

  // ---- this lane's four pixel slots: LDS address of tap (r, 0) (static) and output offset (per tile) ----
  int rowbase[3][4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    unsigned s = (unsigned)(pg * kSlots + j * 32 + lrow);
    const unsigned live = TH * W;
    if (s >= live) {  // a slot without a pixel reads with the last slot that has one and sits a multiple of 16 before it
      const unsigned back = (((s - live) >> 4) + 1u) << 4;
      s = s >= back ? s - back : 0u;
    }
    const unsigned ty = (s * a.t.mW16) >> 16, tx = s - ty * W;
#pragma unroll
    for (int r = 0; r < 3; ++r) rowbase[r][j] = (int)(ty + r) * RPB + (int)tx * kPitchS + (lchunk + 2 * wk * KPG) * 16;
  }
  const int f0 = fb * BF + wf * 32 + 16 * lchunk;    // this lane's 16 consecutive output channels
  unsigned obase[NOWN];  // of the slot groups wk*NOWN .. +NOWN-1, the ones this wave finishes
  auto tile_outputs = [&](int t) {
    const unsigned v0 = top + (unsigned)t * TH;
#pragma unroll
    for (int j = 0; j < NOWN; ++j) {
      const unsigned s = (unsigned)(pg * kSlots + (wk * NOWN + j) * 32 + lrow);
      const unsigned ty = (s * a.t.mW16) >> 16, tx = s - ty * W;
      const unsigned v = v0 + ty;
      const unsigned n = __umulhi(v, a.mS32);
      const unsigned y = v - n * S - top;
      const unsigned bad = (unsigned)(ty >= TH) | (unsigned)(y >= H) | (unsigned)(n >= N);
      const unsigned pixel = (n * H + y) * W + tx;
      obase[j] = ((pixel * (unsigned)a.t.ldo + (unsigned)f0) * 2u) | (bad ? kOOBs : 0u);
    }
  };
  tile_outputs(tile);

  floatx16 acc[4];
  // the first patch is older than the kW - 3 fragments and the two scale / shift loads requested after it
  __builtin_amdgcn_s_waitcnt(vmcnt_only(kW - 1));
  __syncthreads();

  int stage_no = 0;
  int cur = 0;      // LDS offset of the buffer the taps read
  int wo = 0;       // byte offset of the current stage's first iteration in the weight stream
  u32x4 pr[2][4];   // pixel operands of two K steps

  for (;;) {
    const int next_tile = tile + tstep;
    for (int slab = 0; slab < nslab; ++slab) {
      const bool last = RES || slab + 1 == nslab;
      // The patch of the next stage goes into the other buffer.  After the last tile the same instructions
      // are issued with descriptors of no bytes (same count on every path; no memory traffic).
      // the cell offsets of the next tile's patch replace this tile's once its last slab has been requested
      if (last) patch_tile(next_tile, next_tile < tend);
      patch_begin(last ? 0 : slab + 1, cur ^ kPatchB);
      u32x4 rv[NOWN][2];
      // The two workgroups of a CU take turns at the higher wave priority, stage by stage (the first 256 workgroups of
      // a launch are the first on their CUs, more or less).  Left alone the arbiter favours the older wave of a SIMD all
      // the way, the younger workgroup finishes long after the older one and runs the end of its taps alone, where
      // one wave per SIMD keeps the matrix pipe about 60 % busy: 10.4 against 10.7 us on 28x28x128 at batch 32.
      if constexpr (PG == 1 && WK == 2) {
        if (((bid >> 8) ^ (unsigned)stage_no) & 1u) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
        ++stage_no;
      }
      __builtin_amdgcn_sched_barrier(0);
      int wo_next = wo + 9 * 4096;
      if (wo_next >= wwrap) wo_next = 0;

      // ---- taps: 9*KPG K steps, fully unrolled; pixel operands one step ahead, weights kRing steps ahead.
      //      A wave issues in order and about one instruction per eight cycles: four MFMAs in a row followed by
      //      everything else make a step last the sum of both.  So every MFMA is followed by its share of the
      //      step's other work (the read of the next step's pixel operand, a part of a patch piece, the weight
      //      refill), pinned there by scheduling fences, and runs under it. ----
      auto ldp1 = [&](auto step_c, int j) {
        constexpr int st = decltype(step_c)::value;
        constexpr int t = st / KPG, k = st % KPG;
        pr[st & 1][j] = *reinterpret_cast<const u32x4*>(smem + rowbase[t / 3][j] + (t % 3) * kPitchS + k * 32);
      };
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (PG == 1 || j < nrows) ldp1(std::integral_constant<int, 0>(), j);
      auto steps = [&](auto self, auto step_c) -> void {
        constexpr int st = decltype(step_c)::value;
        if constexpr (st < kSteps) {
          constexpr int PPS = (kLoadsPerWave + kPieceSteps - 1) / kPieceSteps;  // patch pieces per step: 1 or 2
          constexpr int nx = st + kRing, nt = nx / KPG, nk = nx % KPG;
          static_assert(nt < 18, "the ring reaches at most into the next stage");
          const u32x4 wfrag = wring[RES ? st : st % kRing];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bool rowlive = PG == 1 || j < nrows;  // a pixel group may hold fewer rows (uniform per wave)
            if (!rowlive) {
            } else if (st == 0 && slab == 0) {
              // the first step of a tile starts the sums: a zero C operand instead of 64 cleared registers
              const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, wfrag), __builtin_bit_cast(half8, pr[st & 1][j]), zero, 0, 0, 0);
            } else {
              Mma<half_t>::run(wfrag, pr[st & 1][j], acc[j]);
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (st + 1 < kSteps) {
              if (rowlive) ldp1(std::integral_constant<int, st + 1>(), j);
            }
            // the next patch: kLoadsPerWave pieces, their permutes over the first kPieceSteps K steps of the stage,
            // each load one step behind its permute
            if constexpr (st * PPS < kLoadsPerWave) {
              if (j == 0) patch_piece_perm(std::integral_constant<int, st * PPS>());
              if constexpr (PPS == 2 && st * PPS + 1 < kLoadsPerWave) {
                if (j == 2) patch_piece_perm(std::integral_constant<int, st * PPS + 1>());
              }
            }
            if constexpr (st >= 1 && (st - 1) * PPS < kLoadsPerWave) {
              if (j == 1) patch_piece_load(std::integral_constant<int, (st - 1) * PPS>());
              if constexpr (PPS == 2 && (st - 1) * PPS + 1 < kLoadsPerWave) {
                if (j == 3) patch_piece_load(std::integral_constant<int, (st - 1) * PPS + 1>());
              }
            }
            // the residual rows this wave finishes go out in the tile's last stage, behind the patch pieces (no
            // residual: a buffer of no bytes, the loads return zeros without touching memory)
            if constexpr (st == kPieceSteps + 1) {
              if (j < NOWN && last) {
                rv[j % NOWN][0] = __builtin_amdgcn_raw_buffer_load_b128(rs_res, obase[j % NOWN], 0, 0);
                rv[j % NOWN][1] = __builtin_amdgcn_raw_buffer_load_b128(rs_res, obase[j % NOWN], 16, 0);
              }
            }
            if (j == 3 && !RES) {
              // refill this ring slot with the fragment kRing steps further down the stream
              if constexpr (nt < 9) {
                wring[st % kRing] = wload_at(wo + nt * 4096 + nk * 1024);
              } else {
                wring[st % kRing] = wload_at(wo_next + (nt - 9) * 4096 + nk * 1024);
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          self(self, std::integral_constant<int, st + 1>());
        }
      };
      steps(steps, std::integral_constant<int, 0>());
      wo = wo_next;

      // The next patch (requested before this stage's kSteps >= kRing weight refills) must have landed, and
      // every wave must be past its taps, before the buffers change roles.
      __builtin_amdgcn_sched_barrier(0);
      if (ss_pending) {
        asm volatile("" : "+v"(vsc), "+v"(vsh));  // keeps this arithmetic (and its wait for the two loads) here
        const float one = a.t.scale ? 0.0f : 1.0f;  // added to the zeros of a missing scale vector
        floatx4 ssv;
#pragma unroll
        for (int q = 0; q < 4; ++q) ssv[q] = ss_shift ? vsh[q] : vsc[q] + one;
        *reinterpret_cast<floatx4*>(smem + 2 * kPatchB + sse * 16) = ssv;
        ss_pending = false;
      }
      __builtin_amdgcn_s_waitcnt(vmcnt_only(kYoung));
      __syncthreads();
      const int done = cur;  // the buffer this stage's taps read: free until the end of the next stage's request
      const int delta = cur ? -kPatchB : kPatchB;
      cur ^= kPatchB;
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int j = 0; j < 4; ++j) rowbase[r][j] += delta;
      if (!last) continue;

      // ---- end of a tile: K groups exchange partial sums through the buffer the taps just left, then
      //      scale/shift, residual, activation, one rounding, two 16-byte stores per pixel ----
      constexpr int FPL = 16;
      if constexpr (WK > 1) {
        // Wave (wf, wk) finishes slot groups [wk*NOWN, (wk+1)*NOWN); the other groups' partial sums go to
        // their owners, lane-linear (kilobytes of 64 lanes x 16 bytes: no bank conflicts, no address math).
        // Two rounds when the partial sums of all four groups do not fit one patch buffer (WK = 4).
        constexpr int NR = WK == 4 ? 2 : 1;
        unsigned char* xb = smem + done;
#pragma unroll
        for (int round = 0; round < NR; ++round) {
          if (round > 0) __syncthreads();  // the previous round's readers are done
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int owner = j / NOWN;
            if ((NR == 1 || j / 2 == round) && owner != wk && (PG == 1 || j < nrows)) {
              const int rank = wk < owner ? wk : wk - 1;  // position among the WK-1 senders
              const int jx = NR == 1 ? j : (j & 1), nj = NR == 1 ? 4 : 2;
              unsigned char* dst = xb + ((((pg * WF + wf) * nj + jx) * (WK - 1) + rank) * 4) * 1024 + lane * 16;
#pragma unroll
              for (int q = 0; q < 4; ++q)
                *reinterpret_cast<floatx4*>(dst + q * 1024) = floatx4{acc[j][4 * q], acc[j][4 * q + 1], acc[j][4 * q + 2], acc[j][4 * q + 3]};
            }
          }
          __syncthreads();
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (j / NOWN == wk && (NR == 1 || j / 2 == round) && (PG == 1 || j < nrows)) {
              const int jx = NR == 1 ? j : (j & 1), nj = NR == 1 ? 4 : 2;
              const unsigned char* src = xb + ((((pg * WF + wf) * nj + jx) * (WK - 1)) * 4) * 1024 + lane * 16;
#pragma unroll
              for (int r = 0; r < WK - 1; ++r)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const floatx4 p = *reinterpret_cast<const floatx4*>(src + (r * 4 + q) * 1024);
#pragma unroll
                  for (int e = 0; e < 4; ++e) acc[j][4 * q + e] += p[e];
                }
            }
          }
        }
      }
      if constexpr (RES) {
        // Without refills nothing younger than the residual rows' loads is ever waited for: on the paths that do not
        // read them (no residual -- the loads still go out, against a descriptor of no bytes -- or a slot group of
        // another wave) they would stay pending in the compiler's books, and the next tile's first reuse of their
        // registers would wait for everything in flight, this tile's stores included.  A use here settles them on
        // every path.
#pragma unroll
        for (int o = 0; o < NOWN; ++o) asm volatile("" : "+v"(rv[o][0]), "+v"(rv[o][1]));
      }
      floatx4 sc4[4], sh4[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        sc4[q] = *reinterpret_cast<const floatx4*>(smem + 2 * kPatchB + (wf * 32 + 16 * lchunk + 4 * q) * 4);
        sh4[q] = *reinterpret_cast<const floatx4*>(smem + 2 * kPatchB + (BF + wf * 32 + 16 * lchunk + 4 * q) * 4);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j / NOWN != wk || (PG > 1 && j >= nrows)) continue;
        const int o = j % NOWN;
        float y[FPL];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) y[4 * q + e] = acc[j][4 * q + e] * sc4[q][e] + sh4[q][e];
        const bool res_after = ACT && (a.t.act & kActResidualAfter);
        float rf[FPL];
        if (a.t.residual) {
          const half8 r0 = __builtin_bit_cast(half8, rv[o][0]), r1 = __builtin_bit_cast(half8, rv[o][1]);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            rf[e] = (float)r0[e];
            rf[8 + e] = (float)r1[e];
          }
          if (!res_after) {
#pragma unroll
            for (int e = 0; e < FPL; ++e) y[e] += rf[e];
          }
        }
        if (a.t.act == kActRelu) {
#pragma unroll
          for (int e = 0; e < FPL; ++e) y[e] = relu_ugt(y[e]);
        } else if (ACT && a.t.act) {
          act_apply_n<true>(y, a.t.act & 0xff);
        }
        if (a.t.residual && res_after) {
#pragma unroll
          for (int e = 0; e < FPL; ++e) y[e] += rf[e];
        }
        half8 o0, o1;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          o0[e] = (half_t)y[e];
          o1[e] = (half_t)y[8 + e];
        }
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o0), rs_out, obase[o], 0, 0);
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o1), rs_out, obase[o], 16, 0);
      }
      if constexpr (WK > 1) __syncthreads();  // the exchange buffer takes a patch again at the start of the next stage
    }
    if (next_tile >= tend) break;
    tile = next_tile;
    tile_outputs(tile);
  }
}

// ---- host side: tile plan ---------------------------------------------------------------------------

struct StreamGeom {
  int TH = 0, NSEG = 0, S = 0, top = 0, aligned = 0, n_tiles = 0;
  int rowx = 0;  // spare bytes behind the segments of a patch row in LDS
};

unsigned recip32(unsigned d) { return d == 1 ? 0u : (unsigned)(0xffffffffull / d + 1); }  // ceil(2^32 / d) for d >= 2

// TH consecutive virtual rows of W columns per tile: at most `slots` pixels, and a patch of TH + 2 rows of
// NSEG segments within `segcap`.  Aligned form: S = bands * TH >= H virtual rows per image, tiles never
// leave their image.  Gap form: S = H + 1 (one shared zero row between images), tiles of the largest TH
// that fits.  The form with fewer tiles wins; aligned on a tie (it wastes no slot on the zero rows).
bool stream_geometry(int N, int H, int W, int slots, int segcap, StreamGeom* g) {
  if (N < 1 || H < 1 || W < 1 || W > slots || H > 254 || N >= (1 << 24)) return false;
  const int NSEG = (W + 2 + kSegCells - 1) / kSegCells;
  int thmax = 0;
  for (int th = 1; th <= H + 1; ++th)
    if (th * W <= slots && (th + 2) * NSEG <= segcap) thmax = th;
  if (thmax == 0) return false;
  const int tha0 = std::min(thmax, H);
  const int bands = (H + tha0 - 1) / tha0, tha = (H + bands - 1) / bands;
  const long long tiles_a = (long long)N * bands;
  const long long rows_g = (long long)N * (H + 1) - 1;  // virtual rows 1 .. N*(H+1)-1
  const long long tiles_g = (rows_g + thmax - 1) / thmax;
  const bool gap = tiles_g < tiles_a;
  g->NSEG = NSEG;
  // The pitch of a patch row in 16-byte units is 9 W mod 16: the slot after the last pixel of a row then reads the bank
  // group after that pixel's, like a neighbour in the row.  At least one unit (the last lane of the row's last load
  // instruction writes it).  When that outgrows the buffer (every segment a wave may load needs a place, also the ones
  // below the patch) the rows stay segments alone, with the bank conflicts that brings.
  {
    const int units = NSEG * (kSegB / 16) + 1, pad = ((9 * W - units) % 16 + 16) % 16;
    g->rowx = 16 * (1 + pad);
    if (segcap * kSegB + ((segcap - 1) / NSEG) * g->rowx + 16 > segcap * kSegB + 64 + kRowPadB) g->rowx = 0;
  }
  if (gap) {
    g->TH = thmax; g->S = H + 1; g->top = 1; g->aligned = 0; g->n_tiles = (int)tiles_g;
  } else {
    g->TH = tha; g->S = bands * tha; g->top = 0; g->aligned = 1; g->n_tiles = (int)tiles_a;
  }
  if (g->S < 2 || g->S > 255) return false;  // the reciprocal of 1 does not exist; S travels in 8 bits
  // the reciprocal multiplications are exact while x * d < 2^32 (x the dividend, d the divisor)
  const long long vmax = (long long)N * g->S + g->TH + 2;
  return (gap ? tiles_g : tiles_a) < (1ll << 24) && vmax * g->S < (1ll << 31);
}

// 3x3 weights FCHW -> the stream kernel's order: per 32-filter group, per 128-byte channel slab, per tap,
// four kilobyte fragments (K sub-steps), each the 64 lanes' 16-byte MFMA A operands in lane order.
// Row rho = 8q + 4h + e of the MFMA holds filter 16h + 4q + e of the group, so that the accumulator
// registers of a lane are 16 consecutive filters.  Filters beyond F are zero.
template <typename Ts>
__global__ void weight_frag32_kernel(const Ts* __restrict__ w, half_t* __restrict__ dst, int F, int C, int Fp) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // one 16-byte chunk each
  const int nslab = C / 64;
  const long long total = (long long)(Fp / 32) * nslab * 9 * 4 * 64;
  if (idx >= total) return;
  const int L = (int)(idx & 63);
  long long r = idx >> 6;
  const int kk = (int)(r & 3); r >>= 2;
  const int tap = (int)(r % 9); r /= 9;
  const int sl = (int)(r % nslab);
  const int g = (int)(r / nslab);
  const int rho = L & 31;
  const int f = g * 32 + 16 * ((rho >> 2) & 1) + 4 * (rho >> 3) + (rho & 3);
  const int c0 = sl * 64 + ((L >> 5) + 2 * kk) * 8;
  half_t* d = dst + idx * 8;
#pragma unroll
  for (int e = 0; e < 8; ++e) d[e] = f < F ? (half_t)(float)w[((long long)f * C + c0 + e) * 9 + tap] : (half_t)0.0f;
}


// The launch shape for a layer: pixel groups, filter groups and K groups of a workgroup, the tile geometry that goes
// with them, and how the (filter block, tile list) pairs spread over the workgroups.
struct StreamConfig {
  int PG = 1, WF = 2, WK = 2;
  StreamGeom geo;
  int FB = 0;        // filter blocks of 32*WF
  int Wpf = 0;       // workgroups per filter block = tile step of a workgroup
  long long cost = 0;
};

// Candidates: four waves, two workgroups per CU -- 128 slots x 64 filters x 2 K groups, or x 32 filters x 4 K groups
// when that is what it takes to fill the CUs; eight waves, one workgroup per CU -- 256 slots x 64 filters x 2 K groups.
// The estimate is the matrix work of the busiest CU: its tiles x the tile's 32-slot rows x filter groups x K steps
// (what the SIMDs of a CU share), plus a per-tile constant for the epilogue.  `only_pg` > 0 restricts the choice.
bool stream_config(int N, int H, int W, int C, int F, bool act, int only_pg, StreamConfig* best) {
  bool found = false;
  static const int force_wf = [] {
    const char* e = getenv("NNCV_HIP_STREAM_WF");
    return e ? atoi(e) : 0;
  }();
  for (int cand = 0; cand < (act ? 2 : 4); ++cand) {  // the eight-wave form and the 128-filter one exist with the ReLU epilogue only
    StreamConfig c;
    c.PG = cand == 2 ? 2 : 1;
    c.WF = cand == 1 ? 1 : cand == 3 ? 4 : 2;
    c.WK = 4 / c.WF;
    if (force_wf > 0 && c.WF != force_wf && !act) continue;
    // Measured, the eight-wave form loses to two independent workgroups of four (13.5 against 12.2 us on 28x28x128 at
    // batch 32): its barriers stop both waves of every SIMD at once, where two workgroups drift apart and fill each
    // other's waits.  It runs on request only (NNCV_HIP_STREAM_PG=2).
    if (c.PG != (only_pg > 0 ? only_pg : 1)) continue;
    if (F % (32 * c.WF) != 0) continue;
    const int nw = 4 * c.PG;
    if (!stream_geometry(N, H, W, kSlots * c.PG, seg_cap(nw), &c.geo)) continue;
    c.FB = F / (32 * c.WF);
    const int per_cu = c.PG == 1 ? 2 : 1;
    // as many workgroups per filter block as the CUs hold, evened out so that all of them walk the same number of
    // tiles (896 tiles on 512 places: 448 workgroups of two tiles, not 384 of two and 128 of one)
    // A one-slab layer in the 64-filter form keeps its weights in registers (RES): the longer a workgroup lives, the
    // fewer fragments cross the vector-memory path.  With passes in flight, where a launch need not fill the chip on
    // its own, its tiles go to half the places (ResNet-18's layer1 at batch 32, four passes in flight, same box: 448
    // workgroups of two tiles 207.5 k images/s, 299 of three 211.9 k, 224 of four 212.6 k, 180 of five 213.2 k,
    // 128 of seven 193 k; one pass at a time the 224 cost 2 % of the pass).
    const bool resident = C == 64 && c.WF == 2 && c.PG == 1 && !act;
    const int per_cu_places = (resident && overlap_hint() >= 3) ? 128 * per_cu : 256 * per_cu;
    const int places = std::max(1, per_cu_places / c.FB), rounds = (c.geo.n_tiles + places - 1) / places;
    c.Wpf = (c.geo.n_tiles + rounds - 1) / rounds;
    const long long wgs = (long long)c.FB * c.Wpf;
    const long long wg_per_cu = (wgs + 255) / 256;  // on the busiest CU
    const int trows = (c.geo.TH * W + 31) / 32;
    const long long ksteps = (long long)C / 64 * 36;
    c.cost = wg_per_cu * rounds * ((long long)trows * c.WF * ksteps + 600);
    // 128 filters per workgroup, no K groups: no exchange of partial sums at the end of a tile.  Measured against the
    // 64-filter form on 28x28x128: 18.1 / 66.4 us against 18.8 / 68.5 at batch 64 / 256 (448 / 512 workgroups).  With
    // about one workgroup per CU (224 at batch 32; 214 on 14x14x256 at batch 64) it is ahead on some runs (10.4 against
    // 10.5, 16.6 against 17.2) and far behind on others (13.9), depending on where the workgroups land, and with 108
    // (14x14x256 at batch 32) it loses outright (15.0 against 10.2): it is taken from 400 workgroups up, and from 160
    // where a tile walks four slabs or more (14x14x256, same box, three runs each: 160 workgroups at batch 48 15.6
    // against 17.8 us, 214 at batch 64 18.1 against 19.2, 320 at batch 96 31.2 against 32.5).
    // When the caller keeps three or more passes in flight it is taken wherever it fits: half the workgroups hold the
    // CUs' slots for about the same time (four passes in flight, ResNet-18 at batch 32: 0.163 against 0.168 ms per pass).
    if (c.WF == 4) c.cost = (wgs >= 400 || (wgs >= 160 && C >= 256) || overlap_hint() >= 3) ? 0 : (1ll << 60);
    if (!found || c.cost < best->cost) {
      *best = c;
      found = true;
    }
  }
  return found;
}

int stream_force_pg() {
  static const int v = [] {
    const char* e = getenv("NNCV_HIP_STREAM_PG");
    return e ? atoi(e) : 0;
  }();
  return v;
}

}  // namespace


size_t weight_frag32_bytes(int F, int C) { return (size_t)((F + 31) / 32) * 32 * 9 * C * 2; }

void launch_weight_frag32(const void* w, int w_dt, void* dst, int F, int C, hipStream_t s) {
  NNCV_REQUIRE(C % 64 == 0, "weight_frag32: C must be a multiple of the 128-byte slab");
  const int Fp = (F + 31) / 32 * 32;
  const long long total = (long long)(Fp / 32) * (C / 64) * 9 * 4 * 64;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (w_dt == kF16) hipLaunchKernelGGL((weight_frag32_kernel<half_t>), dim3(grid), dim3(256), 0, s, (const half_t*)w, (half_t*)dst, F, C, Fp);
  else hipLaunchKernelGGL((weight_frag32_kernel<float>), dim3(grid), dim3(256), 0, s, (const float*)w, (half_t*)dst, F, C, Fp);
  NNCV_HIP_CHECK(hipGetLastError());
}

bool conv3x3_stream_plan(int N, int H, int W, int C, int F, int out[14]) {
  StreamConfig c;
  if (!stream_config(N, H, W, C, F, false, 0, &c)) return false;
  const StreamGeom& g = c.geo;
  out[0] = g.TH; out[1] = g.S; out[2] = g.top; out[3] = g.aligned; out[4] = g.n_tiles; out[5] = g.NSEG;
  out[6] = c.PG; out[7] = c.WF; out[8] = c.WK; out[9] = c.FB; out[10] = c.Wpf; out[11] = seg_cap(4 * c.PG);
  out[12] = g.rowx; out[13] = patch_bytes(4 * c.PG);
  return true;
}

bool conv3x3_stream_applicable(const IgemmArgs& a, int in_dt, int out_dt) {
  static const bool off = getenv("NNCV_HIP_NO_STREAM") != nullptr;
  // The deepest layers (eight channel slabs per tile, few pixels) stay with the patch kernel unless asked for: 16.6 us
  // here against 13.1 there on 7x7x512 at batch 32; up to 256 channels this kernel is 5-8 % ahead.
  static const bool all = getenv("NNCV_HIP_STREAM_ALL") != nullptr;
  if (off || in_dt != kF16 || out_dt != kF16 || !a.wt_frag32 || (a.C > 256 && !all)) return false;
  const int pix = a.pix_stride ? a.pix_stride : a.C;
  const bool act_ok = a.relu <= kActRelu || ((a.relu & 0xff) <= kActSigmoid && (a.relu & ~(0xff | kActResidualAfter)) == 0);
  StreamConfig c;
  const bool shape_ok = act_ok && a.aux_f0 == 0 && a.R == 3 && a.S == 3 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 1 && a.pad_w == 1 &&
         a.OH == a.H && a.OW == a.W && a.batch == 1 && a.C % 64 == 0 && a.F % 32 == 0 && pix % 8 == 0 && a.ldo % 8 == 0 && a.ldo >= a.F &&
         (long long)a.N * a.H * a.W * a.ldo * 2 < (1ll << 31) && (long long)a.N * a.H * a.W * pix * 2 < (1ll << 31) &&
         a.in_bytes < kOOBs && (long long)a.F * 9 * a.C * 2 < (1ll << 31) && stream_config(a.N, a.H, a.W, a.C, a.F, a.relu > kActRelu, stream_force_pg(), &c);
  if (!shape_ok) return false;
  // Small launches and poorly filled tiles stay with the patch kernel (measured, stream / patch us): 1x28x28x128 5.7 /
  // 4.9, 4x28x28x128 5.9 / 5.0, 8x14x14x256 7.9 / 6.3 -- 112 workgroups of 32 filters or fewer -- against 8x28x28x128
  // 5.9 / 6.3, 16x14x14x256 7.9 / 8.6, 4x56x56x64 4.9 / 5.4 (216-224 workgroups); rows of 80 pixels fill 80 of a
  // tile's 128 slots: 16x80x80x64 18.2 / 15.7, where the patch kernel cuts the rows into column tiles.
  const long long fine_wgs = (long long)c.geo.n_tiles * (a.F / 32);
  // With three or more passes in flight (overlap_hint) a ReLU layer whose filter count rules out the 128-filter form goes
  // to the patch kernel, whose 256-slot workgroups hold fewer slots for the same work than the 64-filter form here
  // (ResNet-18's layer1 at batch 32, four passes in flight: 0.161 against 0.165 ms per pass) -- unless it is a one-slab
  // layer, whose 64-filter form keeps the weights in registers (204.4 k images/s with layer1 on the patch kernel,
  // 212.6 k here, same box).
  if (!all && overlap_hint() >= 3 && a.relu <= kActRelu && c.WF != 4 && !(a.C == 64 && c.WF == 2 && c.PG == 1)) return false;
  return all || (fine_wgs >= 160 && c.geo.TH * a.W >= 96);
}

template <int PG, int WF, int WK, bool ACT, bool RES = false>
static void launch_stream_cfg(const StreamArgs& a, int grid, double flops, double bytes, const char* tag, hipStream_t s) {
  auto kern = conv3x3_f16_stream_kernel<PG, WF, WK, ACT, RES>;
  constexpr int NW = PG * WF * WK;
  constexpr int smem = 2 * patch_bytes(NW) + 2 * 32 * WF * 4;
  static const bool attr = [&] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return true;
  }();
  (void)attr;
  ProfScope prof(tag, flops, bytes, s);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), smem, s, a.in, a.wf, a.G, a.div, a.mdiv, a.mS32, a.n_tiles, a.tstep_nslab_flags, a.N_TH, a.geom,
                     a.pixB, a.rowx_rnseg, a.t);
}

bool launch_conv3x3_stream(const IgemmArgs& g, hipStream_t s) {
  StreamConfig cfg;
  if (!stream_config(g.N, g.H, g.W, g.C, g.F, g.relu > kActRelu, stream_force_pg(), &cfg)) return false;
  const StreamGeom& geo = cfg.geo;
  const int FB = cfg.FB, Wpf = cfg.Wpf;
  const size_t wbytes = weight_frag32_bytes(g.F, g.C);
  // An XCD's workgroups are neighbours: a contiguous range of tile lists (tiles that share halo rows meet in one
  // L2) with all filter blocks, or -- when the filters outgrow an L2 -- a range of filter blocks with all lists.
  const bool by_filter = FB % kXcds == 0 && wbytes > (2u << 20);
  const int G = FB * Wpf, grid = (G + kXcds - 1) / kXcds * kXcds;
  NNCV_REQUIRE(Wpf < 65536 && g.C / 64 < 256, "conv3x3_stream: tile step / slab count out of range");
  StreamArgs a{};
  const int pix = g.pix_stride ? g.pix_stride : g.C;
  a.in = g.in; a.wf = g.wt_frag32; a.t.out = g.out; a.t.scale = g.scale; a.t.shift = g.shift; a.t.residual = g.residual;
  a.t.F = g.F; a.t.act = g.relu; a.t.ldo = g.ldo;
  a.t.out_bytes = (unsigned)((size_t)g.N * g.H * g.W * g.ldo * 2);
  a.G = (unsigned)G;
  a.div = (unsigned)(by_filter ? Wpf : FB);
  a.mdiv = recip32(a.div);
  a.mS32 = recip32((unsigned)geo.S);
  a.n_tiles = (unsigned)geo.n_tiles;
  a.tstep_nslab_flags = (unsigned)Wpf | ((unsigned)(g.C / 64) << 16) | ((by_filter ? 1u : 0u) << 24) | ((unsigned)geo.aligned << 25) | ((unsigned)geo.top << 26);
  a.N_TH = (unsigned)g.N | ((unsigned)geo.TH << 24);
  a.geom = (unsigned)g.H | ((unsigned)g.W << 8) | ((unsigned)geo.S << 16) | ((unsigned)geo.NSEG << 24);
  a.pixB = (unsigned)pix * 2u;
  a.rowx_rnseg = (unsigned)geo.rowx | (geo.NSEG == 1 ? 0u : (unsigned)(65535 / geo.NSEG + 1) << 16);
  a.t.mW16 = (unsigned)((65536 + g.W - 1) / g.W);
  const double P = (double)g.N * g.H * g.W;
  const double flops = 2.0 * P * g.C * 9.0 * g.F;
  const double bytes = 2.0 * (P * g.C + 9.0 * g.C * g.F + P * g.F * (g.residual ? 2 : 1));
  const bool act = g.relu > kActRelu;
  if (cfg.PG == 2) {
    launch_stream_cfg<2, 2, 2, false>(a, grid, flops, bytes, "conv3x3_stream<f16,2x2x2>", s);
  } else if (cfg.WF == 4) {
    launch_stream_cfg<1, 4, 1, false>(a, grid, flops, bytes, "conv3x3_stream<f16,1x4x1>", s);
  } else if (cfg.WF == 1) {
    if (act) launch_stream_cfg<1, 1, 4, true>(a, grid, flops, bytes, "conv3x3_stream<f16,1x1x4,act>", s);
    else launch_stream_cfg<1, 1, 4, false>(a, grid, flops, bytes, "conv3x3_stream<f16,1x1x4>", s);
  } else {
    if (act) launch_stream_cfg<1, 2, 2, true>(a, grid, flops, bytes, "conv3x3_stream<f16,1x2x2,act>", s);
    else if (g.C == 64) launch_stream_cfg<1, 2, 2, false, true>(a, grid, flops, bytes, "conv3x3_stream<f16,1x2x2,res>", s);
    else launch_stream_cfg<1, 2, 2, false>(a, grid, flops, bytes, "conv3x3_stream<f16,1x2x2>", s);
  }
  NNCV_HIP_CHECK(hipGetLastError());
  return true;
}

}  // namespace nncv_hip
