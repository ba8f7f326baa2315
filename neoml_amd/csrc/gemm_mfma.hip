// fp32 matrix products and channels-last convolution on the CDNA4 matrix cores.
//
// One kernel template serves every dense contraction of the engine:
//   C[M x N] (+)= A * B (+ bias[n])
// with A given K-major (row-major M x K), M-major (a K x M matrix read transposed) or implicitly as the
// im2col view of an N,H,W,C image (K = fh*fw*Cin gathered on the fly, zero padding), and B given K-major
// (N x K, i.e. "multiply by transposed matrix" / the filter blob [Cout][fh][fw][Cin]) or N-major (K x N).
//
// Tiling: 256 threads = 4 wavefronts per workgroup; workgroup tile BM x BN (64x64, or 128x32 for narrow outputs),
// K step 16; each wavefront owns
// a (BM/WAVES_M) x (BN/WAVES_N) sub-tile built from 32x32 blocks of v_mfma_f32_32x32x2_f32 (16 accumulator
// registers per block).
//
// Data path: operands are fetched with raw buffer loads (a 32-bit offset per lane that stays put, plus what a K step
// adds in a scalar register; the memory unit's range check supplies the zeros of padding and of partial tiles),
// parked in registers for one K step, written to one of two LDS buffers (20 KB per workgroup: eight workgroups
// per compute unit) and read back as MFMA operands. Within a wavefront the LDS reads
// of the next group of 8 k are issued before the MFMAs of the current group, and the single barrier of a K step
// sits before its last group, so the matrix pipe of a wavefront does not wait for LDS, barrier or memory in steady
// state.
//
// Small grids: when the tiles alone would leave the compute units with one or two workgroups each, K is cut into
// slices (grid z). The slices of one matrix meet inside the launch through partial tiles in scratch memory, summed
// in slice order by the slice that arrives last; batched products, the gradient by a filter and launches recorded
// into a graph add their partial products into C with fp32 atomics after C has been set to the free term (the
// summation order of those slices varies from run to run, differences at the 1e-7 relative level).
//
// LDS layout for a K-major operand is [row][16 + 4 pad]; lane (row = lane % 32, half = lane / 32) fetches the
// four consecutive k values  k0 + 4*half .. +3  with a single 128-bit LDS read and feeds them to four MFMAs.
// MFMA j of a group therefore reduces over k = {k0 + j, k0 + 4 + j}; both operands use the same permutation of
// k, which is all the dot product needs.
#include "common.h"
#include <math.h>
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

namespace nh {

typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );

// AM_Conv1x1 runs the same code as AM_Conv; the separate value gives 1x1 convolutions their own kernel symbols, so
// that profiles tell them apart from the 3x3 ones
// AM_ConvRows serves channel counts that are not a multiple of 4 (grey and RGB inputs): the reduction index runs
// over Fh filter rows of RowPitch = ceil4( Fw * Cin ) values each. The Fw * Cin values that one filter row meets are
// contiguous in a channels-last image (no dilation along the width), so they are fetched as 128-bit runs however
// Cin divides; the 1-3 padding values per row are masked to zero on both operands.
// AM_ConvClasses: the gradient by the input of a strided convolution, one stride-1 convolution per residue class of the
// input pixels (blockIdx.y = class): AM_Conv whose geometry, filter and output rows come from args.Class[class].
// AM_ConvTaps: AM_Conv for channel counts that are a multiple of the K step, without the strided gradient's exact-division
// test: a step never straddles two taps, the reduction ends on a step, and everything that is only needed otherwise is
// compiled out of the loop ( the 3x3 convolutions of the image networks ).
enum TAMode { AM_RowsK = 0, AM_RowsM = 1, AM_Conv = 2, AM_Conv1x1 = 3, AM_ConvRows = 4, AM_ConvClasses = 5, AM_ConvTaps = 6 };
// BM_ConvN: B is the im2col view of an N,H,W,C image read N-major: row k = output pixel, column n = ( kh, kw, ci ).
// With A = the gradient by the convolution's output read M-major this is the gradient by the filter.
enum TBMode { BM_RowsK = 0, BM_RowsN = 1, BM_ConvN = 2 };

// One residue class ( ( hi + pad ) mod stride, same along the width ) of the input pixels of a strided convolution. Only
// the filter taps kh with kh * dilation in the same class reach its pixels, Fh x Fw of them, and through them the
// class is a stride-1 convolution over the output gradient. Its result rows are the pixels
// ( OutH0 + j * strideH, OutW0 + i * strideW ), j < Ho, i < Wo, of every image.
struct CConvClass {
	int K, Fh, Fw, PadH, PadW, Ho, Wo, M, OutH0, OutW0;
	long long BOffset; // of the class's filter [N][Fh][Fw][Cin] inside B, in floats
};

constexpr int MaxConvClasses = 4;

struct CMatMulArgs {
	const float* A;
	const float* B;
	float* C;
	const float* Bias; // per column n, may be null
	int M, N, K;
	int Lda, Ldb, Ldc;
	long long BatchStrideA, BatchStrideB, BatchStrideC;
	int Accumulate; // C += instead of C =
	int SplitK;     // number of K slices (grid z); > 1: partial products are added to C with atomics
	int StepsPerSplit;
	int TilesM, TilesN;
	// convolution geometry (AM_Conv only): A is the image, M = batch * Ho * Wo
	int H, W, Cin, Ho, Wo, Fh, Fw, PadH, PadW, StrideH, StrideW, DilH, DilW;
	int RowK, RowPitch; // AM_ConvRows: Fw * Cin and its round-up to a multiple of 4; K = Fh * RowPitch
	int AFloats, BFloats; // AM_ConvRows: sizes of the image and of the filter, the limit of a 128-bit load that reads past a run
	// AM_Conv as the gradient by the input of a strided convolution: the tap's source coordinate is
	// ( ho * StrideH - PadH + kh * DilH ) / UpH and only exists where that division is exact (values <= 1: no division)
	int UpH, UpW;
	int ManySlices; // the reduction is far longer than the output is large: as many K slices as fill the device
	// Tail mode (FullTiles > 0, grid z = 1): the first FullTiles workgroups compute one whole tile each; the workgroups
	// behind them share the TailTiles remaining tiles, TailSplit slices of TailSteps K steps per tile, and meet in C
	// through atomic adds like the K slices above
	int FullTiles, TailTiles, TailSplit, TailSteps;
	// K slices that meet without atomics (Partials != null): every slice leaves its accumulators in Partials
	// [ sliced tile ][ slice ][ 4096 ] and counts itself in Counters[ sliced tile ]; the slice that counts last adds
	// them up in slice order, runs the ordinary epilogue and sets the counter back to zero for the next launch.
	float* Partials;
	unsigned* Counters;
	// AM_ConvClasses: the dense result is [images][OutH][OutW][Ldc], DenseM pixels in all
	int OutH, OutW, OutUpH, OutUpW, DenseM;
	CConvClass Class[MaxConvClasses];
	// epilogue of the fused blocks: C = act( A * B + bias ) + Residual; Residual has C's layout, may be C itself
	CFusedActivation Act;
	const float* Residual;
	// floor( 2^32 / divisor ) for the divisions of the prologue ( pixel -> image, row, column; workgroup -> tile ): a
	// multiplication and one correction instead of the twenty-odd instructions of a division by a run-time value
	unsigned WoMagic, HoMagic, TilesNMagic;
	// size of C in bytes when its rows can be addressed by 32-bit offsets from its start ( 0: they cannot ): the
	// epilogue then stores through a buffer descriptor of that size, which drops the rows of a last tile that lie
	// beyond the matrix by itself
	unsigned CBytes;
};

// floor( 2^32 / d ), capped: with it q = mulhi( x, magic ) is floor( x / d ) or one less for every x < 2^32
inline unsigned divisionMagic( int d )
{
	return d <= 1 ? 0xFFFFFFFFu : static_cast<unsigned>( 0x100000000ULL / static_cast<unsigned>( d ) );
}

__device__ __forceinline__ void fastDivMod( int x, int d, unsigned magic, int& quotient, int& remainder )
{
	unsigned q = __umulhi( static_cast<unsigned>( x ), magic );
	unsigned r = static_cast<unsigned>( x ) - q * static_cast<unsigned>( d );
	const bool low = r >= static_cast<unsigned>( d );
	quotient = static_cast<int>( low ? q + 1 : q );
	remainder = static_cast<int>( low ? r - static_cast<unsigned>( d ) : r );
}

constexpr int Threads = 256;

#ifndef NH_KSTEP
#define NH_KSTEP 16
#endif

// KGROUPS == 2: the workgroup has two groups of 4 wavefronts; each group runs the whole pipeline on its own LDS buffers
// over one half of the K steps of the tile, then the second group hands its accumulators to the first through LDS.
// For problems of a few hundred tiles with a reduction long enough to cut in two: the same number of waves per compute
// unit as two K slices in separate workgroups, without the preset of C, the atomics and the separate activation pass.
template<int BM, int BN, int WAVES_M, int WAVES_N, int AMODE, int BMODE, bool VEC, int KGROUPS = 1>
__global__ __launch_bounds__( Threads * KGROUPS, KGROUPS == 1 ? 2 : 1 )
void matMulKernel( const CMatMulArgs launchArgs )
{
	constexpr bool IsClasses = ( AMODE == AM_ConvClasses );
	CMatMulArgs args = launchArgs;
	int outH0 = 0, outW0 = 0;
	if constexpr( IsClasses ) {
		const CConvClass& c = launchArgs.Class[blockIdx.y];
		args.K = c.K; args.Ldb = c.K; args.B += c.BOffset;
		args.Fh = c.Fh; args.Fw = c.Fw; args.PadH = c.PadH; args.PadW = c.PadW;
		args.Ho = c.Ho; args.Wo = c.Wo; args.M = c.M;
		outH0 = c.OutH0; outW0 = c.OutW0;
	}
	constexpr int KS = NH_KSTEP;           // K step per pipeline stage
	constexpr int KQ = KS / 4;             // float4 slots along K of a K-major tile row
	constexpr int LdsK = KS + 4;           // row pitch of a K-major tile in LDS
	static_assert( WAVES_M * WAVES_N == 4, "4 wavefronts per workgroup" );
	constexpr int WM = BM / WAVES_M;
	constexpr int WN = BN / WAVES_N;
	constexpr int MI = WM / 32;
	constexpr int NI = WN / 32;
	constexpr bool AK = ( AMODE != AM_RowsM );
	constexpr bool IsTaps = ( AMODE == AM_ConvTaps );
	constexpr bool IsConv = ( AMODE == AM_Conv || AMODE == AM_Conv1x1 || AMODE == AM_ConvClasses || IsTaps );
	static_assert( !IsTaps || VEC, "whole taps per step go with vector loads" );
	constexpr bool IsConvRows = ( AMODE == AM_ConvRows );
	constexpr bool BK = ( BMODE == BM_RowsK );
	constexpr int APitchX = BM + 4, BPitchX = BN + 4;
	constexpr int ASize = AK ? BM * LdsK : KS * APitchX;
	constexpr int BSize = BK ? BN * LdsK : KS * BPitchX;
	constexpr int ATotal = BM * KQ, BTotal = BN * KQ; // float4 slots per tile
	constexpr int ASlots = ( ATotal + Threads - 1 ) / Threads;
	constexpr int BSlots = ( BTotal + Threads - 1 ) / Threads;

	__shared__ __attribute__( ( aligned( 16 ) ) ) float lds[KGROUPS][2][ASize + BSize];

	const int kGroup = KGROUPS == 1 ? 0 : __builtin_amdgcn_readfirstlane( threadIdx.x / Threads ); // same for a whole wave
	const int tid = KGROUPS == 1 ? threadIdx.x : threadIdx.x % Threads; // inside the group
	auto ldsA = [&]( int buf ) -> float* { return lds[kGroup][buf]; };
	auto ldsB = [&]( int buf ) -> float* { return lds[kGroup][buf] + ASize; };
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int waveM = wave / WAVES_N;
	const int waveN = wave % WAVES_N;
	const int l32 = lane & 31;
	const int half = lane >> 5;

	int tile = xcdSwizzle( blockIdx.x, gridDim.x );
	int split = blockIdx.z;
	int splitK = args.SplitK, stepsPerSplit = args.StepsPerSplit;
	if( args.FullTiles > 0 ) {
		if( blockIdx.x < args.FullTiles ) {
			tile = xcdSwizzle( blockIdx.x, args.FullTiles );
		} else {
			const int j = blockIdx.x - args.FullTiles;
			split = j / args.TailTiles;
			tile = args.FullTiles + ( j - split * args.TailTiles );
			splitK = args.TailSplit;
			stepsPerSplit = args.TailSteps;
		}
	}
	int tileM, tileN;
	fastDivMod( tile, args.TilesN, args.TilesNMagic, tileM, tileN );
	const int m0 = tileM * BM;
	const int n0 = tileN * BN;
	const int batch = blockIdx.y;

	const float* A = args.A + batch * args.BatchStrideA;
	const float* B = args.B + batch * args.BatchStrideB;
	float* C = args.C + batch * args.BatchStrideC;
	const int M = args.M, N = args.N, K = args.K;
	if constexpr( KGROUPS == 2 ) {
		// the launch has one slice ( split == 0 ) of an even number of steps: this group's half of it
		stepsPerSplit = ( ( K + NH_KSTEP - 1 ) / NH_KSTEP ) / 2;
		split = kGroup;
	}
	const int kStart = split * stepsPerSplit * NH_KSTEP; // first k of this workgroup's K slice
	if constexpr( IsClasses ) {
		// classes differ in their row and reduction counts; the grid is sized for the largest
		if( m0 >= M || ( split > 0 && kStart >= K ) ) {
			return;
		}
	}
	const __amdgpu_buffer_rsrc_t bufA = makeBuffer( A );
	const __amdgpu_buffer_rsrc_t bufB = makeBuffer( B );

	// ---- per-thread load slots ---------------------------------------------------------------------------
	// K-major tile: slot -> ( row = rowOfSlot( slot ), kq = slot % KQ ); X-major tile: slot -> ( k = slot / (BX/4), xq ).
	// The rows of a K-major tile are dealt to the slots so that the two rows which eight consecutive lanes write with
	// one 128-bit LDS store are four rows apart: at a pitch of 20 floats they then cover all 32 banks once ( rows next to
	// each other share four banks, which doubles the time of every store ). Memory still sees 64 contiguous bytes per row.
	auto rowOfSlot = []( int slot ) -> int {
		const int q = slot / KQ;
		return ( q & ~7 ) | ( ( q & 1 ) << 2 ) | ( ( q & 6 ) >> 1 );
	};
	// Vector path: offA / offB hold the byte offset of the slot for the K step that is loaded next.
	unsigned offA[ASlots], offB[BSlots];
	int convPixel[ASlots], convH0[ASlots], convW0[ASlots];
	int convCi = 0, convKh = 0, convKw = 0;

	auto convSlotOffset = [&]( int i ) -> unsigned {
		int hi = convH0[i] + convKh * args.DilH;
		int wi = convW0[i] + convKw * args.DilW;
		bool ok = convKh < args.Fh;
		if( !IsTaps && ( args.UpH > 1 || args.UpW > 1 ) ) {
			ok = ok && hi >= 0 && wi >= 0 && hi % args.UpH == 0 && wi % args.UpW == 0;
			hi /= args.UpH;
			wi /= args.UpW;
		}
		ok = ok && hi >= 0 && hi < args.H && wi >= 0 && wi < args.W;
		return ok ? static_cast<unsigned>( convPixel[i] + ( hi * args.W + wi ) * args.Cin + convCi ) * 4u : OutOfRange;
	};

#pragma unroll
	for( int i = 0; i < ASlots; ++i ) {
		const int slot = tid + i * Threads;
		const bool inTile = ATotal % Threads == 0 || slot < ATotal;
		if( AMODE == AM_RowsK ) {
			const int m = m0 + rowOfSlot( slot );
			offA[i] = ( inTile && m < M ) ? static_cast<unsigned>( m * args.Lda + kStart + ( slot % KQ ) * 4 ) * 4u : OutOfRange;
		} else if( AMODE == AM_RowsM ) {
			const int m = m0 + ( slot % ( BM / 4 ) ) * 4;
			offA[i] = ( inTile && m < M ) ? static_cast<unsigned>( ( kStart + slot / ( BM / 4 ) ) * args.Lda + m ) * 4u : OutOfRange;
		} else {
			const int m = m0 + rowOfSlot( slot );
			if( inTile && m < M ) {
				int wo, t, ho, n;
				if constexpr( IsClasses ) {
					// ( every class has its own grid of result pixels )
					wo = m % args.Wo;
					t = m / args.Wo;
					ho = t % args.Ho;
					n = t / args.Ho;
				} else {
					fastDivMod( m, args.Wo, args.WoMagic, t, wo );
					fastDivMod( t, args.Ho, args.HoMagic, n, ho );
				}
				convPixel[i] = n * args.H * args.W * args.Cin;
				convH0[i] = ho * args.StrideH - args.PadH;
				convW0[i] = ( wo * args.StrideW - args.PadW ) * ( IsConvRows ? args.Cin : 1 ); // AM_ConvRows: in floats

			} else {
				convPixel[i] = 0;
				convH0[i] = -0x40000000; // never inside the image
				convW0[i] = 0;
			}
		}
	}
	// AM_ConvRows: filter row and position inside the padded row of this thread's k (all its slots share the column)
	int rowKh = 0, rowR = 0;
	if( IsConvRows ) {
		const int k = kStart + ( tid % KQ ) * 4;
		rowKh = k / args.RowPitch;
		rowR = k - rowKh * args.RowPitch;
	}
	// Channel counts that are a multiple of the K step: every lane of the workgroup is in the same filter tap during a
	// step, so the tap and the channel inside it live in scalar registers, the channel reaches the loads as their
	// uniform offset, and a step inside a tap costs no vector instruction for addresses.
	const bool uniformTap = IsTaps || ( IsConv && VEC && args.Cin % KS == 0 );
	int tapCi = 0, tapKh = 0, tapKw = 0;
	// Without the strided gradient's division a tap moves every lane's address by the same amount: per slot the position
	// of tap ( 0, 0 ) is kept ( in floats, as unsigned arithmetic: it may lie in front of the image ), a tap adds
	// ( kh dilation W + kw dilation ) Cin from a scalar register, and the two unsigned comparisons say whether the tap
	// meets the image: six vector instructions per slot and tap.
	unsigned convBase[ASlots] = {};
#pragma unroll
	for( int i = 0; IsConv && i < ASlots; ++i ) {
		convBase[i] = static_cast<unsigned>( convPixel[i] ) + ( static_cast<unsigned>( convH0[i] ) * static_cast<unsigned>( args.W )
			+ static_cast<unsigned>( convW0[i] ) ) * static_cast<unsigned>( args.Cin ) + static_cast<unsigned>( ( tid % KQ ) * 4 );
	}
	auto tapSlotOffset = [&]( int i ) -> unsigned {
		if( !IsTaps && ( args.UpH > 1 || args.UpW > 1 ) ) {
			int hi = convH0[i] + tapKh * args.DilH;
			int wi = convW0[i] + tapKw * args.DilW;
			bool ok = tapKh < args.Fh && hi >= 0 && wi >= 0 && hi % args.UpH == 0 && wi % args.UpW == 0;
			hi /= args.UpH;
			wi /= args.UpW;
			ok = ok && hi >= 0 && hi < args.H && wi >= 0 && wi < args.W;
			return ok ? static_cast<unsigned>( convPixel[i] + ( hi * args.W + wi ) * args.Cin + ( tid % KQ ) * 4 ) * 4u : OutOfRange;
		}
		const int dh = tapKh * args.DilH, dw = tapKw * args.DilW; // ( scalar )
		const unsigned tapFloats = ( static_cast<unsigned>( dh ) * static_cast<unsigned>( args.W ) + static_cast<unsigned>( dw ) )
			* static_cast<unsigned>( args.Cin );
		const bool ok = tapKh < args.Fh && static_cast<unsigned>( convH0[i] + dh ) < static_cast<unsigned>( args.H )
			&& static_cast<unsigned>( convW0[i] + dw ) < static_cast<unsigned>( args.W );
		return ok ? ( convBase[i] + tapFloats ) * 4u : OutOfRange;
	};
	if( IsConv && VEC ) {
		if( uniformTap ) {
			if( kStart != 0 ) { // ( a slice behind the first: the only case that pays for the two divisions )
				const int tap = kStart / args.Cin;
				tapCi = kStart - tap * args.Cin;
				tapKh = tap / args.Fw;
				tapKw = tap - tapKh * args.Fw;
			}
#pragma unroll
			for( int i = 0; i < ASlots; ++i ) {
				offA[i] = tapSlotOffset( i );
			}
		} else {
			const int k = kStart + ( tid % KQ ) * 4;
			const int tap = k / args.Cin;
			convCi = k - tap * args.Cin;
			convKh = tap / args.Fw;
			convKw = tap - convKh * args.Fw;
#pragma unroll
			for( int i = 0; i < ASlots; ++i ) {
				offA[i] = convSlotOffset( i );
			}
		}
	}
	// BM_ConvN: per slot, the tap of its four columns ( fixed for the whole launch ) and the output pixel of its row
	// ( advances by KS pixels per K step )
	int bDh[BSlots], bDw[BSlots], bCi[BSlots], bImg[BSlots], bHo[BSlots], bWo[BSlots];
	long long bPixel[BSlots];
#pragma unroll
	for( int i = 0; i < BSlots; ++i ) {
		const int slot = tid + i * Threads;
		const bool inTile = BTotal % Threads == 0 || slot < BTotal;
		if( BMODE == BM_ConvN ) {
			const int n = n0 + ( slot % ( BN / 4 ) ) * 4;
			const bool nOk = inTile && n < N;
			if( args.RowPitch > 0 ) {
				// channel counts that are not a multiple of 4: column n = kh * RowPitch + r, r = position inside the run of
				// Fw * Cin values that a filter row meets in an image row ( r >= RowK: padding of the run, dropped on output )
				const int kh = n / args.RowPitch;
				bCi[i] = n - kh * args.RowPitch;
				bDh[i] = nOk ? kh * args.DilH - args.PadH : -0x40000000; // never inside the image
				bDw[i] = bCi[i] - args.PadW * args.Cin; // in floats, from the image row's position of the output column
			} else {
				const int tap = n / args.Cin;
				bCi[i] = n - tap * args.Cin;
				const int kh = tap / args.Fw;
				bDh[i] = nOk ? kh * args.DilH - args.PadH : -0x40000000; // never inside the image
				bDw[i] = ( tap - kh * args.Fw ) * args.DilW - args.PadW;
			}
			const long long pixel = static_cast<long long>( kStart ) + slot / ( BN / 4 );
			bPixel[i] = pixel;
			bWo[i] = static_cast<int>( pixel % args.Wo );
			const long long t = pixel / args.Wo;
			bHo[i] = static_cast<int>( t % args.Ho );
			bImg[i] = static_cast<int>( t / args.Ho );
			offB[i] = 0;
		} else if( BMODE == BM_RowsK ) {
			const int n = n0 + rowOfSlot( slot );
			offB[i] = ( inTile && n < N ) ? static_cast<unsigned>( n * args.Ldb + kStart + ( slot % KQ ) * 4 ) * 4u : OutOfRange;
		} else {
			const int n = n0 + ( slot % ( BN / 4 ) ) * 4;
			offB[i] = ( inTile && n < N ) ? static_cast<unsigned>( ( kStart + slot / ( BN / 4 ) ) * args.Ldb + n ) * 4u : OutOfRange;
		}
	}

	auto loadConvElement = [&]( int i, int k ) -> float {
		if( k >= K ) {
			return 0.f;
		}
		const int tap = k / args.Cin;
		const int ci = k - tap * args.Cin;
		const int kh = tap / args.Fw;
		const int kw = tap - kh * args.Fw;
		int hi = convH0[i] + kh * args.DilH;
		int wi = convW0[i] + kw * args.DilW;
		if( args.UpH > 1 || args.UpW > 1 ) {
			if( hi < 0 || wi < 0 || hi % args.UpH != 0 || wi % args.UpW != 0 ) {
				return 0.f;
			}
			hi /= args.UpH;
			wi /= args.UpW;
		}
		if( hi < 0 || hi >= args.H || wi < 0 || wi >= args.W ) {
			return 0.f;
		}
		return A[convPixel[i] + ( hi * args.W + wi ) * args.Cin + ci];
	};

	// im2col element ( output pixel, column n ) of the image B, zero outside (BM_ConvN, scalar path)
	auto loadIm2colElement = [&]( long long pixel, int n ) -> float {
		if( pixel >= K || n >= N ) {
			return 0.f;
		}
		const int wo = static_cast<int>( pixel % args.Wo );
		const long long t = pixel / args.Wo;
		const int ho = static_cast<int>( t % args.Ho );
		const long long img = t / args.Ho;
		const int tap = n / args.Cin;
		const int ci = n - tap * args.Cin;
		const int kh = tap / args.Fw;
		const int kw = tap - kh * args.Fw;
		const int hi = ho * args.StrideH - args.PadH + kh * args.DilH;
		const int wi = wo * args.StrideW - args.PadW + kw * args.DilW;
		if( hi < 0 || hi >= args.H || wi < 0 || wi >= args.W ) {
			return 0.f;
		}
		return B[( ( img * args.H + hi ) * args.W + wi ) * args.Cin + ci];
	};

	// Loads the tiles of the K step starting at kBase into registers and advances the slot offsets to the next step.
	auto loadTiles = [&]( int kBase, float4 ( &regA )[ASlots], float4 ( &regB )[BSlots] ) {
		if constexpr( IsConvRows ) {
			const int rowFloats = args.W * args.Cin;
			const bool khIn = rowKh < args.Fh;
			// A run that ends inside these four values ( the last values of a filter row, the right edge of the image ) is
			// still fetched with one 128-bit load, as long as the load stays inside the tensor, and the values beyond the
			// run's end are replaced by zeros: what lies there is the next pixels, not padding. Only a run that BEGINS inside
			// the four values ( the left edge ) or touches the tensor's end is fetched value by value.
			const int leftInRow = args.RowK - rowR; // values of the filter row from this lane's k on; <= 0 in the padding of K
			auto maskTail = []( float4 v, int valid ) -> float4 {
				return make_float4( v.x, valid > 1 ? v.y : 0.f, valid > 2 ? v.z : 0.f, valid > 3 ? v.w : 0.f );
			};
#pragma unroll
			for( int i = 0; i < ASlots; ++i ) {
				const int hi = convH0[i] + rowKh * args.DilH;
				const bool rowOk = khIn && hi >= 0 && hi < args.H;
				const int col = convW0[i] + rowR; // position inside the image row, in floats; negative in the left padding
				const int index = convPixel[i] + hi * rowFloats + col;
				const int valid = min( leftInRow, rowFloats - col );
				if( !rowOk || valid <= 0 || col <= -4 ) {
					regA[i] = make_float4( 0.f, 0.f, 0.f, 0.f );
				} else if( col >= 0 && index + 3 < args.AFloats ) {
					regA[i] = maskTail( bufferLoad4( bufA, static_cast<unsigned>( index ) * 4u ), valid );
				} else {
					float v[4];
#pragma unroll
					for( int e = 0; e < 4; ++e ) {
						const bool ok = e < valid && col + e >= 0;
						v[e] = bufferLoad1( bufA, ok ? static_cast<unsigned>( index + e ) * 4u : OutOfRange );
					}
					regA[i] = make_float4( v[0], v[1], v[2], v[3] );
				}
			}
#pragma unroll
			for( int i = 0; i < BSlots; ++i ) {
				const int slot = tid + i * Threads;
				const int n = n0 + rowOfSlot( slot );
				const bool nOk = ( BTotal % Threads == 0 || slot < BTotal ) && n < N && khIn;
				const int index = n * args.Ldb + rowKh * args.RowK + rowR;
				if( !nOk || leftInRow <= 0 ) {
					regB[i] = make_float4( 0.f, 0.f, 0.f, 0.f );
				} else if( index + 3 < args.BFloats ) {
					regB[i] = maskTail( bufferLoad4( bufB, static_cast<unsigned>( index ) * 4u ), leftInRow );
				} else {
					float v[4];
#pragma unroll
					for( int e = 0; e < 4; ++e ) {
						v[e] = bufferLoad1( bufB, e < leftInRow ? static_cast<unsigned>( index + e ) * 4u : OutOfRange );
					}
					regB[i] = make_float4( v[0], v[1], v[2], v[3] );
				}
			}
			rowR += KS;
			while( rowR >= args.RowPitch ) {
				rowR -= args.RowPitch;
				++rowKh;
			}
			return;
		}
		if( VEC ) {
			// Offsets of the slots stay where the slice begins; what a step adds is the same for every lane and goes to
			// the loads as their uniform offset. Only the last step of a K that is not a multiple of the step masks k.
			const unsigned stepK = static_cast<unsigned>( kBase - kStart );
			const unsigned uniA = IsConv ? ( uniformTap ? static_cast<unsigned>( tapCi ) * 4u : 0u )
				: ( AMODE == AM_RowsK ? stepK * 4u : stepK * static_cast<unsigned>( args.Lda ) * 4u );
			const unsigned uniB = BMODE == BM_ConvN ? 0u
				: ( BMODE == BM_RowsK ? stepK * 4u : stepK * static_cast<unsigned>( args.Ldb ) * 4u );
			const bool partialStep = !IsTaps && kBase + KS > K; // ( whole taps of whole steps: K ends on a step )
			if( IsConv || !partialStep ) {
				// the image's own zero padding covers k beyond K: such taps lie below the filter ( kh >= Fh )
#pragma unroll
				for( int i = 0; i < ASlots; ++i ) {
					regA[i] = bufferLoad4( bufA, offA[i], uniA );
				}
			} else {
				asm volatile( "" ); // keeps this rare case a branch of its own instead of selects in every step
#pragma unroll
				for( int i = 0; i < ASlots; ++i ) {
					const int kOfSlot = AMODE == AM_RowsM ? ( tid + i * Threads ) / ( BM / 4 ) : ( tid % KQ ) * 4;
					regA[i] = bufferLoad4( bufA, kBase + kOfSlot < K ? offA[i] : OutOfRange, uniA );
				}
			}
			if( BMODE == BM_ConvN ) {
#pragma unroll
				for( int i = 0; i < BSlots; ++i ) {
					const int hi = bHo[i] * args.StrideH + bDh[i];
					if( args.RowPitch > 0 ) {
						// four values of a filter row's run in the image row: one 128-bit load at 4-byte alignment whose
						// values beyond the run's end or the row's end are replaced by zeros; element-wise only where the
						// run begins inside the four ( left edge ) or the load would leave the tensor
						const int rowFloats = args.W * args.Cin;
						const int col = bWo[i] * args.StrideW * args.Cin + bDw[i];
						const bool rowOk = bPixel[i] < K && hi >= 0 && hi < args.H;
						const int valid = min( args.RowK - bCi[i], rowFloats - col );
						const int index = ( bImg[i] * args.H + hi ) * rowFloats + col;
						if( !rowOk || valid <= 0 || col <= -4 ) {
							regB[i] = make_float4( 0.f, 0.f, 0.f, 0.f );
						} else if( col >= 0 && index + 3 < args.BFloats ) {
							const float4 v = bufferLoad4( bufB, static_cast<unsigned>( index ) * 4u );
							regB[i] = make_float4( v.x, valid > 1 ? v.y : 0.f, valid > 2 ? v.z : 0.f, valid > 3 ? v.w : 0.f );
						} else {
							float v[4];
#pragma unroll
							for( int e = 0; e < 4; ++e ) {
								v[e] = bufferLoad1( bufB, ( e < valid && col + e >= 0 ) ? static_cast<unsigned>( index + e ) * 4u : OutOfRange );
							}
							regB[i] = make_float4( v[0], v[1], v[2], v[3] );
						}
					}
					const int wi = bWo[i] * args.StrideW + bDw[i];
					const bool ok = bPixel[i] < K && hi >= 0 && hi < args.H && wi >= 0 && wi < args.W;
					const unsigned off = ok ? static_cast<unsigned>( ( ( bImg[i] * args.H + hi ) * args.W + wi ) * args.Cin + bCi[i] ) * 4u : OutOfRange;
					// the row of this slot in the next K step
					bPixel[i] += KS;
					bWo[i] += KS;
					while( bWo[i] >= args.Wo ) {
						bWo[i] -= args.Wo;
						if( ++bHo[i] == args.Ho ) {
							bHo[i] = 0;
							++bImg[i];
						}
					}
					if( args.RowPitch <= 0 ) {
						regB[i] = bufferLoad4( bufB, off );
					}
				}
			} else if( !partialStep ) {
#pragma unroll
				for( int i = 0; i < BSlots; ++i ) {
					regB[i] = bufferLoad4( bufB, offB[i], uniB );
				}
			} else {
				asm volatile( "" );
#pragma unroll
				for( int i = 0; i < BSlots; ++i ) {
					const int kOfSlot = BMODE == BM_RowsK ? ( tid % KQ ) * 4 : ( tid + i * Threads ) / ( BN / 4 );
					regB[i] = bufferLoad4( bufB, kBase + kOfSlot < K ? offB[i] : OutOfRange, uniB );
				}
			}
			// advance the convolution's tap
			if( IsConv ) {
				if( uniformTap ) {
					tapCi += KS;
					if( tapCi >= args.Cin ) {
						tapCi = 0;
						if( ++tapKw == args.Fw ) {
							tapKw = 0;
							++tapKh;
						}
#pragma unroll
						for( int i = 0; i < ASlots; ++i ) {
							offA[i] = tapSlotOffset( i );
						}
					}
				} else {
					convCi += KS;
					if( convCi >= args.Cin ) {
						do {
							convCi -= args.Cin;
							if( ++convKw == args.Fw ) {
								convKw = 0;
								++convKh;
							}
						} while( convCi >= args.Cin );
#pragma unroll
						for( int i = 0; i < ASlots; ++i ) {
							offA[i] = convSlotOffset( i );
						}
					} else {
#pragma unroll
						for( int i = 0; i < ASlots; ++i ) {
							offA[i] += KS * 4;
						}
					}
				}
			}
			return;
		}
		// scalar path: any alignment, any shape
#pragma unroll
		for( int i = 0; i < ASlots; ++i ) {
			const int slot = tid + i * Threads;
			float4 v = make_float4( 0.f, 0.f, 0.f, 0.f );
			if( ATotal % Threads == 0 || slot < ATotal ) {
				if( AMODE == AM_RowsK ) {
					const int m = m0 + rowOfSlot( slot );
					const int k = kBase + ( slot % KQ ) * 4;
					if( m < M ) {
						const float* p = A + static_cast<long long>( m ) * args.Lda + k;
						if( k < K ) v.x = p[0];
						if( k + 1 < K ) v.y = p[1];
						if( k + 2 < K ) v.z = p[2];
						if( k + 3 < K ) v.w = p[3];
					}
				} else if( AMODE == AM_RowsM ) {
					const int k = kBase + slot / ( BM / 4 );
					const int m = m0 + ( slot % ( BM / 4 ) ) * 4;
					if( k < K ) {
						const float* p = A + static_cast<long long>( k ) * args.Lda + m;
						if( m < M ) v.x = p[0];
						if( m + 1 < M ) v.y = p[1];
						if( m + 2 < M ) v.z = p[2];
						if( m + 3 < M ) v.w = p[3];
					}
				} else {
					const int k = kBase + ( slot % KQ ) * 4;
					v.x = loadConvElement( i, k );
					v.y = loadConvElement( i, k + 1 );
					v.z = loadConvElement( i, k + 2 );
					v.w = loadConvElement( i, k + 3 );
				}
			}
			regA[i] = v;
		}
#pragma unroll
		for( int i = 0; i < BSlots; ++i ) {
			const int slot = tid + i * Threads;
			float4 v = make_float4( 0.f, 0.f, 0.f, 0.f );
			if( BTotal % Threads == 0 || slot < BTotal ) {
				if( BMODE == BM_RowsK ) {
					const int n = n0 + rowOfSlot( slot );
					const int k = kBase + ( slot % KQ ) * 4;
					if( n < N ) {
						const float* p = B + static_cast<long long>( n ) * args.Ldb + k;
						if( k < K ) v.x = p[0];
						if( k + 1 < K ) v.y = p[1];
						if( k + 2 < K ) v.z = p[2];
						if( k + 3 < K ) v.w = p[3];
					}
				} else if( BMODE == BM_ConvN ) {
					const long long pixel = static_cast<long long>( kBase ) + slot / ( BN / 4 );
					const int n = n0 + ( slot % ( BN / 4 ) ) * 4;
					v.x = loadIm2colElement( pixel, n );
					v.y = loadIm2colElement( pixel, n + 1 );
					v.z = loadIm2colElement( pixel, n + 2 );
					v.w = loadIm2colElement( pixel, n + 3 );
				} else {
					const int k = kBase + slot / ( BN / 4 );
					const int n = n0 + ( slot % ( BN / 4 ) ) * 4;
					if( k < K ) {
						const float* p = B + static_cast<long long>( k ) * args.Ldb + n;
						if( n < N ) v.x = p[0];
						if( n + 1 < N ) v.y = p[1];
						if( n + 2 < N ) v.z = p[2];
						if( n + 3 < N ) v.w = p[3];
					}
				}
			}
			regB[i] = v;
		}
	};

	auto storeTiles = [&]( int buf, const float4 ( &regA )[ASlots], const float4 ( &regB )[BSlots] ) {
#pragma unroll
		for( int i = 0; i < ASlots; ++i ) {
			const int slot = tid + i * Threads;
			if( ATotal % Threads == 0 || slot < ATotal ) {
				if( AK ) {
					*reinterpret_cast<float4*>( &ldsA( buf )[rowOfSlot( slot ) * LdsK + ( slot % KQ ) * 4] ) = regA[i];
				} else {
					*reinterpret_cast<float4*>( &ldsA( buf )[( slot / ( BM / 4 ) ) * APitchX + ( slot % ( BM / 4 ) ) * 4] ) = regA[i];
				}
			}
		}
#pragma unroll
		for( int i = 0; i < BSlots; ++i ) {
			const int slot = tid + i * Threads;
			if( BTotal % Threads == 0 || slot < BTotal ) {
				if( BK ) {
					*reinterpret_cast<float4*>( &ldsB( buf )[rowOfSlot( slot ) * LdsK + ( slot % KQ ) * 4] ) = regB[i];
				} else {
					*reinterpret_cast<float4*>( &ldsB( buf )[( slot / ( BN / 4 ) ) * BPitchX + ( slot % ( BN / 4 ) ) * 4] ) = regB[i];
				}
			}
		}
	};

	f32x16 acc[MI][NI];
#pragma unroll
	for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
		for( int ni = 0; ni < NI; ++ni ) {
#pragma unroll
			for( int r = 0; r < 16; ++r ) {
				acc[mi][ni][r] = 0.f;
			}
		}
	}

	// Fragments of one group of 8 k values: four MFMA operands per 32-row block of A and of B.
	struct CFrag {
		float A[MI][4];
		float B[NI][4];
	};
	auto readFrag = [&]( int buf, int kc, CFrag& f ) {
		const float* tA = ldsA( buf );
		const float* tB = ldsB( buf );
#pragma unroll
		for( int mi = 0; mi < MI; ++mi ) {
			const int row = waveM * WM + mi * 32 + l32;
			if( AK ) {
				const float4 v = *reinterpret_cast<const float4*>( &tA[row * LdsK + kc * 8 + half * 4] );
				f.A[mi][0] = v.x; f.A[mi][1] = v.y; f.A[mi][2] = v.z; f.A[mi][3] = v.w;
			} else {
#pragma unroll
				for( int j = 0; j < 4; ++j ) {
					f.A[mi][j] = tA[( kc * 8 + half * 4 + j ) * APitchX + row];
				}
			}
		}
#pragma unroll
		for( int ni = 0; ni < NI; ++ni ) {
			const int col = waveN * WN + ni * 32 + l32;
			if( BK ) {
				const float4 v = *reinterpret_cast<const float4*>( &tB[col * LdsK + kc * 8 + half * 4] );
				f.B[ni][0] = v.x; f.B[ni][1] = v.y; f.B[ni][2] = v.z; f.B[ni][3] = v.w;
			} else {
#pragma unroll
				for( int j = 0; j < 4; ++j ) {
					f.B[ni][j] = tB[( kc * 8 + half * 4 + j ) * BPitchX + col];
				}
			}
		}
	};
	auto multiply = [&]( const CFrag& f ) {
#pragma unroll
		for( int j = 0; j < 4; ++j ) {
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
				for( int ni = 0; ni < NI; ++ni ) {
					acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32( f.A[mi][j], f.B[ni][j], acc[mi][ni], 0, 0, 0 );
				}
			}
		}
	};

	// Software pipeline over K steps of KS, two LDS buffers, one barrier per step:
	//   top of step ks : the tiles of step ks+1 (loaded from memory during step ks-1) go to LDS buffer (ks+1)%2, then
	//                    the loads of step ks+2 are issued;
	//   body           : the MFMAs of each group of 8 k run while the fragments of the following group are being
	//                    read from LDS; the barrier sits before the last group, after which the first fragments of
	//                    step ks+1 are fetched, so neither the LDS latency nor the barrier leaves the MFMA pipe idle.
	// Buffer (ks+1)%2 was last read in step ks-1 BEFORE that step's barrier (the fragments of a step's last group are
	// fetched ahead of the barrier, and a wave waits for its LDS reads before it enters the barrier; behind the barrier
	// a wave only reads the other buffer), and a wave that stores at the top of step ks has passed that barrier: two
	// buffers are enough, and the smaller footprint puts eight workgroups instead of five on a compute unit.
	const int totalSteps = ( K + KS - 1 ) / KS;
	const int kSteps = min( stepsPerSplit, totalSteps - split * stepsPerSplit );
	constexpr int Groups = KS / 8;
	// Two sets of load registers: the operands of step ks + 1 wait in set ( ks + 1 ) % 2 while those of step ks + 2 are on
	// their way into the other set, so a load has two steps' time before its values are needed. The steps are unrolled
	// by two ( set and LDS buffer are compile-time constants ), and the steady state is a loop of its own in which every
	// step stores and reloads unconditionally: the wait in front of the store then counts exactly the loads of the
	// other set as still outstanding.
	float4 rA[2][ASlots], rB[2][BSlots];
	CFrag frag[2];
	// a class without taps ( kSteps == 0 ) only writes the free term
	auto step = [&]( int ks, auto setOf, auto steadyOf ) {
		constexpr int set = decltype( setOf )::value; // == ( ks + 1 ) % 2: register set of step ks + 1 and the LDS buffer it goes to
		constexpr bool steady = decltype( steadyOf )::value;
		constexpr int cur = set ^ 1, nxt = set;
		if( steady || ks + 1 < kSteps ) {
			storeTiles( nxt, rA[set], rB[set] );
		}
		if( steady || ks + 3 < kSteps ) {
			loadTiles( kStart + ( ks + 3 ) * KS, rA[set], rB[set] );
		}
		__builtin_amdgcn_sched_barrier( 0 );
#pragma unroll
		for( int g = 0; g < Groups; ++g ) {
			if( g + 1 < Groups ) {
				readFrag( cur, g + 1, frag[( g + 1 ) & 1] );
			} else {
				__syncthreads();
				if( steady || ks + 1 < kSteps ) {
					readFrag( nxt, 0, frag[( g + 1 ) & 1] );
				}
			}
			__builtin_amdgcn_sched_barrier( 0 );
			multiply( frag[g & 1] );
			__builtin_amdgcn_sched_barrier( 0 );
		}
	};
	int ks = 0;
	const bool hasSteadySteps = kSteps > 4;
	if( hasSteadySteps ) {
		// ( a branch of its own: on the way into the steady loop every one of these loads has been issued, which is what
		// lets the waits in that loop leave the younger set's loads outstanding )
		loadTiles( kStart, rA[0], rB[0] );
		storeTiles( 0, rA[0], rB[0] );
		loadTiles( kStart + KS, rA[1], rB[1] );
		loadTiles( kStart + 2 * KS, rA[0], rB[0] );
		__syncthreads();
		readFrag( 0, 0, frag[0] );
		asm volatile( "; into the steady loop" ); // keeps this path apart from the one below up to the loop
		for( ; ks + 4 < kSteps; ks += 2 ) {
			step( ks, std::integral_constant<int, 1>(), std::true_type() );
			step( ks + 1, std::integral_constant<int, 0>(), std::true_type() );
		}
	} else if( !IsClasses || kSteps > 0 ) {
		loadTiles( kStart, rA[0], rB[0] );
		storeTiles( 0, rA[0], rB[0] );
		if( kSteps > 1 ) {
			loadTiles( kStart + KS, rA[1], rB[1] );
		}
		if( kSteps > 2 ) {
			loadTiles( kStart + 2 * KS, rA[0], rB[0] );
		}
		__syncthreads();
		readFrag( 0, 0, frag[0] );
	}
	static_assert( Groups % 2 == 0, "the fragment buffers are back where they started after a step" );
	for( ; ks < kSteps; ks += 2 ) {
		step( ks, std::integral_constant<int, 1>(), std::false_type() );
		if( ks + 1 < kSteps ) {
			step( ks + 1, std::integral_constant<int, 0>(), std::false_type() );
		}
	}

	if constexpr( KGROUPS == 2 ) {
		// every wave has passed the last barrier of its loop behind its last LDS read: the buffers are free
		float* hand = &lds[1][0][0] + wave * ( MI * NI * 16 * 64 ) + lane;
		if( kGroup == 1 ) {
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
				for( int ni = 0; ni < NI; ++ni ) {
#pragma unroll
					for( int r = 0; r < 16; ++r ) {
						hand[( ( mi * NI + ni ) * 16 + r ) * 64] = acc[mi][ni][r];
					}
				}
			}
		}
		__syncthreads();
		if( kGroup == 1 ) {
			return;
		}
#pragma unroll
		for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
			for( int ni = 0; ni < NI; ++ni ) {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					acc[mi][ni][r] += hand[( ( mi * NI + ni ) * 16 + r ) * 64];
				}
			}
		}
	}

	if constexpr( MI * NI == 1 && KGROUPS == 1 ) {
		if( splitK > 1 && args.Partials != nullptr ) {
			// Values cross between workgroups (and so between the L2 caches of the XCDs) through device-scope atomic
			// stores and loads, which go past those caches. A wave's stores are complete when the barrier lets it
			// through, the count follows the barrier: whoever reads the full count finds every slice's values.
			// Why relaxed operations are enough here, and what holds them in place:
			//  - every access to the partial tiles and to the counter is an agent-scope ATOMIC: the compiler may neither
			//    drop, merge nor cache one, and emits each as an access that is coherent across the XCDs ( write-through
			//    stores, loads that miss the XCD's L2 ), so no cache has to be written back or invalidated;
			//  - the partial stores cannot sink below the ticket: between them lie the explicit wait for the wave's own
			//    stores and __syncthreads(), which is a workgroup-scope release fence, the barrier, and an acquire fence;
			//    the fences order ALL earlier memory operations of the wave, atomic or not, before all later ones for the
			//    compiler, and the wait makes the hardware's stores complete ( acknowledged by the memory side ) first;
			//  - the last arriver's loads cannot rise above the ticket: they come behind the second __syncthreads() and
			//    depend on the ticket's value through the branch.
			// A release on the ticket and an acquire in front of the loads would say the same in the language's terms; at
			// agent scope they make this part write back and invalidate the XCD's whole L2, result tiles of other
			// workgroups included: measured once, an acq_rel ticket took the K-sliced 3x3 convolutions from 122 / 127 /
			// 123 us to 145 / 166 / 159 us ( 64 x 28 x 28 x 128, 64 x 14 x 14 x 256, 64 x 7 x 7 x 512 ).
			const int slicedTile = args.FullTiles > 0 ? tile - args.FullTiles : tile;
			unsigned* mine = reinterpret_cast<unsigned*>( args.Partials )
				+ ( static_cast<long long>( slicedTile ) * splitK + split ) * ( BM * BN ) + wave * 64 + lane;
#pragma unroll
			for( int r = 0; r < 16; ++r ) {
				__hip_atomic_store( mine + r * Threads, __float_as_uint( acc[0][0][r] ), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
			}
			__builtin_amdgcn_s_waitcnt( 0x0F70 ); // vmcnt( 0 ): this wave's stores have been acknowledged
			__syncthreads();
			unsigned* arrived = reinterpret_cast<unsigned*>( &lds[0][0][0] );
			if( tid == 0 ) {
				*arrived = __hip_atomic_fetch_add( args.Counters + slicedTile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
			}
			__syncthreads();
			if( *arrived != static_cast<unsigned>( splitK - 1 ) ) {
				return;
			}
			f32x16 total;
#pragma unroll
			for( int r = 0; r < 16; ++r ) {
				total[r] = 0.f;
			}
			const unsigned* first = mine - static_cast<long long>( split ) * ( BM * BN );
			for( int slice = 0; slice < splitK; ++slice ) {
				if( slice == split ) {
#pragma unroll
					for( int r = 0; r < 16; ++r ) {
						total[r] += acc[0][0][r];
					}
				} else {
					const unsigned* theirs = first + static_cast<long long>( slice ) * ( BM * BN );
#pragma unroll
					for( int r = 0; r < 16; ++r ) {
						total[r] += __uint_as_float( __hip_atomic_load( theirs + r * Threads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT ) );
					}
				}
			}
			acc[0][0] = total;
			if( tid == 0 ) {
				__hip_atomic_store( args.Counters + slicedTile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
			}
			splitK = 1; // from here on: the one workgroup that writes the tile
		}
	}

	// The common case - C = act( acc + bias ), rows addressable by 32-bit offsets - stores through a buffer descriptor that
	// ends with the matrix: a lane's offset is computed once per 32-column block, a row adds a multiple of the row pitch
	// ( in a scalar register for tiles that lie inside the matrix: no vector instruction per element beyond the bias and
	// the activation; as a vector addition for the last tile row, whose rows beyond M the range check drops ). Per tile
	// and wavefront this takes some 150 vector instructions out of an epilogue that cost as much as ten K steps.
	if constexpr( !IsClasses && BMODE != BM_ConvN ) {
		if( args.CBytes != 0 && splitK == 1 && !args.Accumulate && args.Residual == nullptr ) {
			const __amdgpu_buffer_rsrc_t bufC = __builtin_amdgcn_make_buffer_rsrc( C, 0, args.CBytes, 0x00020000 );
			const float actParam = withParam( args.Act ).Param; // ( the threshold may live in device memory )
			const float reluTop = actParam > 0.f ? actParam : __builtin_inff();
			const unsigned pitchBytes = static_cast<unsigned>( args.Ldc ) * 4u;
			const bool inside = m0 + BM <= M;
			auto store = [&]( auto typeOf, auto insideOf ) {
				constexpr int Type = decltype( typeOf )::value;
				constexpr bool Inside = decltype( insideOf )::value;
#pragma unroll
				for( int ni = 0; ni < NI; ++ni ) {
					const int n = n0 + waveN * WN + ni * 32 + l32;
					const float bias = ( args.Bias != nullptr && n < N ) ? args.Bias[n] : 0.f;
					const unsigned laneOffset = n < N
						? static_cast<unsigned>( ( m0 + waveM * WM + half * 4 ) * args.Ldc + n ) * 4u : OutOfRange;
#pragma unroll
					for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
						for( int r = 0; r < 16; ++r ) {
							const unsigned rowBytes = static_cast<unsigned>( mi * 32 + ( r >> 2 ) * 8 + ( r & 3 ) ) * pitchBytes;
							const float v = applyActivationOf<Type>( acc[mi][ni][r] + bias, reluTop );
							if constexpr( Inside ) {
								__builtin_amdgcn_raw_buffer_store_b32( __float_as_uint( v ), bufC, laneOffset, rowBytes, 0 );
							} else {
								// ( an offset that was out of range stays so: rowBytes is below 2^31 )
								__builtin_amdgcn_raw_buffer_store_b32( __float_as_uint( v ), bufC, laneOffset + rowBytes, 0, 0 );
							}
						}
					}
				}
			};
			auto storeAs = [&]( auto typeOf ) {
				if( inside ) {
					store( typeOf, std::true_type() );
				} else {
					store( typeOf, std::false_type() );
				}
			};
			if( args.Act.Type == NH_ACT_RELU ) {
				storeAs( std::integral_constant<int, NH_ACT_RELU>() );
			} else if( args.Act.Type == NH_ACT_HSWISH ) {
				storeAs( std::integral_constant<int, NH_ACT_HSWISH>() );
			} else {
				storeAs( std::integral_constant<int, NH_ACT_NONE>() );
			}
			return;
		}
	}

#pragma unroll
	for( int ni = 0; ni < NI; ++ni ) {
		int n = n0 + waveN * WN + ni * 32 + l32;
		if( n >= N ) {
			continue;
		}
		if( BMODE == BM_ConvN && args.RowPitch > 0 ) {
			// the padded runs of the columns close up: ( kh, r ) -> kh * RowK + r
			const int kh = n / args.RowPitch;
			const int r = n - kh * args.RowPitch;
			if( r >= args.RowK ) {
				continue;
			}
			n = kh * args.RowK + r;
		}
		const float bias = ( args.Bias != nullptr ) ? args.Bias[n] : 0.f;
		const float actParam = withParam( args.Act ).Param; // ( the threshold may live in device memory )
			const float reluTop = actParam > 0.f ? actParam : __builtin_inff();
		// Mode: 0 adds onto C with atomics ( K slices that meet in C: it was set to the free term, or left as it was when
		// accumulating, before the launch ), 1 stores act( acc + bias ), 2 also accumulates and / or adds the residual.
		// What is the same for the whole tile is decided once per tile, not per element: with up to eight wavefronts per SIMD
		// a handful of branches in front of every one of a lane's 16 or 32 stores costs microseconds per launch.
		auto write = [&]( auto modeOf, auto typeOf ) {
			constexpr int Mode = decltype( modeOf )::value;
			constexpr int Type = decltype( typeOf )::value;
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					const int m = m0 + waveM * WM + mi * 32 + ( r >> 2 ) * 8 + half * 4 + ( r & 3 );
					if( m < M ) {
						long long row = m;
						if constexpr( IsClasses ) {
							const int wo = m % args.Wo;
							const int t = m / args.Wo;
							const int ho = t % args.Ho;
							row = ( static_cast<long long>( t / args.Ho ) * args.OutH + outH0 + ho * args.OutUpH ) * args.OutW
								+ outW0 + wo * args.OutUpW;
						}
						float* p = C + row * args.Ldc + n;
						if constexpr( Mode == 0 ) {
							unsafeAtomicAdd( p, acc[mi][ni][r] );
						} else {
							float v = acc[mi][ni][r] + bias;
							if constexpr( Mode == 2 ) {
								if( args.Accumulate ) {
									v += *p;
								}
							}
							v = applyActivationOf<Type>( v, reluTop );
							if constexpr( Mode == 2 ) {
								if( args.Residual != nullptr ) {
									v += args.Residual[batch * args.BatchStrideC + row * args.Ldc + n];
								}
							}
							*p = v;
						}
					}
				}
			}
		};
		auto writeAs = [&]( auto typeOf ) {
			if( args.Accumulate || args.Residual != nullptr ) {
				write( std::integral_constant<int, 2>(), typeOf );
			} else {
				write( std::integral_constant<int, 1>(), typeOf );
			}
		};
		if( splitK > 1 ) {
			write( std::integral_constant<int, 0>(), std::integral_constant<int, NH_ACT_NONE>() );
		} else if( args.Act.Type == NH_ACT_RELU ) {
			writeAs( std::integral_constant<int, NH_ACT_RELU>() );
		} else if( args.Act.Type == NH_ACT_HSWISH ) {
			writeAs( std::integral_constant<int, NH_ACT_HSWISH>() );
		} else {
			writeAs( std::integral_constant<int, NH_ACT_NONE>() );
		}
	}
}

// Scratch of the K slices that meet without atomics: partial tiles and arrival counters, one pair per stream (launches
// of one stream run in order and may share it; two streams must not). Grown on demand by doubling; a block that has been
// outgrown is NOT freed while the stream keeps its scratch: another thread may be about to launch on the same stream with
// the address it was handed a moment ago. All blocks of a stream (together at most twice the largest request) are freed by
// releaseSliceScratch: when the stream is destroyed through nhStreamDestroy, or when its owner asks
// (nhStreamReleaseScratch); those of other streams live until the process ends.
// A stream that has been bound to a caching pool (nhStreamBindPool) takes its blocks from that pool and gives them back
// to it, so the pool's memory limit, statistics and clean-up cover them; other streams use the raw allocator.
// The counters start at zero and every launch leaves them at zero.
struct CSliceScratch {
	float* Partials = nullptr;
	size_t PartialFloats = 0;
	unsigned* Counters = nullptr;
	size_t CounterCount = 0;
	std::vector<void*> Blocks; // every allocation made for the stream
	nhPool Pool = nullptr;     // where the blocks came from; null = the raw allocator
};

static std::mutex sliceScratchLock;
static std::map<std::pair<int, hipStream_t>, CSliceScratch>& sliceScratchByStream()
{
	static std::map<std::pair<int, hipStream_t>, CSliceScratch> byStream;
	return byStream;
}
static std::map<std::pair<int, hipStream_t>, nhPool>& poolByStream()
{
	static std::map<std::pair<int, hipStream_t>, nhPool> byStream;
	return byStream;
}

static void freeSliceBlocks( CSliceScratch& scratch )
{
	for( void* block : scratch.Blocks ) {
		if( scratch.Pool != nullptr ) {
			( void )nhPoolHeapFree( scratch.Pool, block );
		} else {
			( void )hipFree( block );
		}
	}
	scratch = CSliceScratch();
}

void releaseSliceScratch( hipStream_t stream, bool unbind )
{
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return;
	}
	std::lock_guard<std::mutex> guard( sliceScratchLock );
	const std::pair<int, hipStream_t> key = std::make_pair( device, stream );
	auto& byStream = sliceScratchByStream();
	auto found = byStream.find( key );
	if( found != byStream.end() ) {
		freeSliceBlocks( found->second );
		byStream.erase( found );
	}
	if( unbind ) {
		poolByStream().erase( key );
	}
}

int bindSliceScratchPool( hipStream_t stream, nhPool pool )
{
	int device = 0;
	NH_HIP( hipGetDevice( &device ) );
	std::lock_guard<std::mutex> guard( sliceScratchLock );
	const std::pair<int, hipStream_t> key = std::make_pair( device, stream );
	auto& byStream = sliceScratchByStream();
	auto found = byStream.find( key );
	if( found != byStream.end() && found->second.Pool != pool ) {
		// blocks from the previous source go back there ( the caller has drained the stream )
		freeSliceBlocks( found->second );
		byStream.erase( found );
	}
	if( pool != nullptr ) {
		poolByStream()[key] = pool;
	} else {
		poolByStream().erase( key );
	}
	return NH_OK;
}

// hipStreamPerThread names a different queue in every thread: launches of two threads on that handle may run side by
// side, so it never gets a block ( its slices meet through atomic adds ). The null stream and hipStreamLegacy name the
// one legacy queue of the device, whose launches run in order whoever issues them.
static bool isSharedStreamHandle( hipStream_t stream )
{
	return stream == hipStreamPerThread;
}

static bool sliceScratch( hipStream_t stream, size_t partialFloats, size_t counters, CSliceScratch& out )
{
	if( isSharedStreamHandle( stream ) ) {
		return false;
	}
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		return false;
	}
	std::lock_guard<std::mutex> guard( sliceScratchLock );
	auto& byStream = sliceScratchByStream();
	// A recorded graph may replay on another stream, beside launches that use this stream's block: launches under
	// capture take the atomic path.
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipStreamIsCapturing( stream, &capture ) != hipSuccess || capture != hipStreamCaptureStatusNone ) {
		( void )hipGetLastError();
		return false;
	}
	const std::pair<int, hipStream_t> key = std::make_pair( device, stream );
	CSliceScratch& scratch = byStream[key];
	if( scratch.Blocks.empty() ) {
		auto bound = poolByStream().find( key );
		scratch.Pool = bound != poolByStream().end() ? bound->second : nullptr;
	}
	// a pool that cannot give the block ( its memory limit ) is not an error here: the slices then meet through atomics
	auto allocate = [&]( size_t bytes ) -> void* {
		void* block = nullptr;
		if( scratch.Pool != nullptr ) {
			if( nhPoolHeapAlloc( scratch.Pool, bytes, &block ) != NH_OK ) {
				return nullptr;
			}
		} else if( hipMalloc( &block, bytes ) != hipSuccess ) {
			( void )hipGetLastError();
			return nullptr;
		}
		scratch.Blocks.push_back( block );
		return block;
	};
	if( scratch.PartialFloats < partialFloats ) {
		const size_t grown = partialFloats > 2 * scratch.PartialFloats ? partialFloats : 2 * scratch.PartialFloats;
		float* block = static_cast<float*>( allocate( grown * sizeof( float ) ) );
		if( block == nullptr ) {
			return false;
		}
		scratch.Partials = block;
		scratch.PartialFloats = grown;
	}
	if( scratch.CounterCount < counters ) {
		size_t grown = counters > 2 * scratch.CounterCount ? counters : 2 * scratch.CounterCount;
		grown = grown > 4096 ? grown : 4096;
		unsigned* block = static_cast<unsigned*>( allocate( grown * sizeof( unsigned ) ) );
		if( block == nullptr ) {
			return false;
		}
		// cleared on the launch stream, ahead of the launch that first uses it
		if( hipMemsetAsync( block, 0, grown * sizeof( unsigned ), stream ) != hipSuccess ) {
			( void )hipGetLastError();
			return false;
		}
		scratch.Counters = block;
		scratch.CounterCount = grown;
	}
	out.Partials = scratch.Partials;
	out.Counters = scratch.Counters;
	return true;
}

// The same block for other reductions that meet inside a launch ( vector sums ): partial results and one arrival counter,
// which every user leaves at zero. false: none to be had ( a capturing stream, a shared stream handle, no memory ).
bool streamMeetingPlace( hipStream_t stream, size_t partialFloats, float** partials, unsigned** counter )
{
	CSliceScratch scratch;
	if( !sliceScratch( stream, partialFloats, 1, scratch ) ) {
		return false;
	}
	*partials = scratch.Partials;
	*counter = scratch.Counters;
	return true;
}

// A meeting place handed in by the caller instead of the stream's block: the launch neither allocates nor looks the
// stream up, and fails when the place is too small.
struct CSliceMeeting {
	float* Partials;
	size_t PartialFloats;
	unsigned* Counters;
	size_t CounterCount;
};

// The meeting place of nhBlobConvolutionNoAlloc: a fixed array in the library's own device image, one copy per GPU,
// held from the moment the library is loaded on that GPU until the process ends. Partial tiles first, the arrival
// counters behind them. Every call on a GPU shares that GPU's copy, so calls that overlap there race.
constexpr size_t NoAllocPartialFloats = NH_NOALLOC_SCRATCH_BYTES / sizeof( float );
constexpr size_t NoAllocCounters = NH_NOALLOC_MAX_SLICED_TILES;
static __device__ __align__( 256 ) unsigned char scratch[NH_NOALLOC_SCRATCH_BYTES + NoAllocCounters * sizeof( unsigned )];

// The array's address on the current device. In host code the array's name is only a stand-in for the symbol, not a
// device address: the address is asked for once per device, with that device current, and kept.
constexpr int MaxDevices = 64;
static std::mutex noAllocLock;
static unsigned char* noAllocScratch[MaxDevices] = {};

static int noAllocMeeting( CSliceMeeting& meeting )
{
	int device = 0;
	NH_HIP( hipGetDevice( &device ) );
	if( device < 0 || device >= MaxDevices ) {
		setLastError( "nhBlobConvolutionNoAlloc: device index %d is beyond the %d devices the library keeps scratch for", device, MaxDevices );
		return NH_ERR_UNSUPPORTED;
	}
	std::lock_guard<std::mutex> guard( noAllocLock );
	if( noAllocScratch[device] == nullptr ) {
		unsigned char* ptr = nullptr;
		NH_HIP( hipGetSymbolAddress( reinterpret_cast<void**>( &ptr ), HIP_SYMBOL( scratch ) ) );
		NH_REQUIRE( ptr != nullptr );
		noAllocScratch[device] = ptr;
	}
	unsigned char* base = noAllocScratch[device];
	meeting.Partials = reinterpret_cast<float*>( base );
	meeting.PartialFloats = NoAllocPartialFloats;
	meeting.Counters = reinterpret_cast<unsigned*>( base + NH_NOALLOC_SCRATCH_BYTES );
	meeting.CounterCount = NoAllocCounters;
	return NH_OK;
}

// a fill kernel rather than a memset: callers may be recording a graph
__global__ __launch_bounds__( 256 ) void clearCountersKernel( unsigned* counters, int count )
{
	for( int i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256 ) {
		counters[i] = 0u;
	}
}

// C[b][m][n] = bias[n] (or 0): the starting value that the K slices add their partial products to
__global__ __launch_bounds__( 256 ) void presetResultKernel( float* c, const float* bias, int M, int N, int ldc, long long batchStride )
{
	const long long total = static_cast<long long>( M ) * N;
	float* base = c + blockIdx.y * batchStride;
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		const int m = static_cast<int>( i / N );
		const int n = static_cast<int>( i - static_cast<long long>( m ) * N );
		base[static_cast<long long>( m ) * ldc + n] = bias != nullptr ? bias[n] : 0.f;
	}
}

// C[b][m][n] = act( C[b][m][n] ): the activation pass behind a launch that met in C through K slices
__global__ __launch_bounds__( 256 ) void activateResultKernel( float* c, int M, int N, int ldc, long long batchStride, const CFusedActivation actAsGiven )
{
	const CFusedActivation act = withParam( actAsGiven );
	const long long total = static_cast<long long>( M ) * N;
	float* base = c + blockIdx.y * batchStride;
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		const int m = static_cast<int>( i / N );
		const int n = static_cast<int>( i - static_cast<long long>( m ) * N );
		float* p = base + static_cast<long long>( m ) * ldc + n;
		*p = applyActivation( *p, act );
	}
}

// the same for rows that lie back to back ( ldc == N, a multiple of 4, 16-byte aligned ): 128-bit stores, no division per element
__global__ __launch_bounds__( 256 ) void presetDenseResultKernel( float4* c, const float* bias, int N, long long quads )
{
	const int quadsPerRow = N >> 2;
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < quads; i += static_cast<long long>( gridDim.x ) * 256 ) {
		float4 v = make_float4( 0.f, 0.f, 0.f, 0.f );
		if( bias != nullptr ) {
			v = *reinterpret_cast<const float4*>( bias + static_cast<int>( i % quadsPerRow ) * 4 );
		}
		c[i] = v;
	}
}

static int presetResult( hipStream_t stream, const CMatMulArgs& args, int batch )
{
	if( batch == 1 && args.Ldc == args.N && args.N % 4 == 0 && isAligned16( args.C ) && ( args.Bias == nullptr || isAligned16( args.Bias ) ) ) {
		const long long quads = static_cast<long long>( args.M ) * ( args.N / 4 );
		long long blocks = ( quads + 1023 ) / 1024; // four stores per thread
		blocks = blocks > 16384 ? 16384 : ( blocks < 1 ? 1 : blocks );
		hipLaunchKernelGGL( presetDenseResultKernel, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			reinterpret_cast<float4*>( args.C ), args.Bias, args.N, quads );
		NH_LAUNCH_CHECK();
		return NH_OK;
	}
	const long long total = static_cast<long long>( args.M ) * args.N;
	long long blocks = ( total + 1023 ) / 1024;
	blocks = blocks > 4096 ? 4096 : blocks;
	for( int b0 = 0; b0 < batch; b0 += 65535 ) {
		const int nb = batch - b0 < 65535 ? batch - b0 : 65535;
		hipLaunchKernelGGL( presetResultKernel, dim3( static_cast<unsigned>( blocks ), nb ), dim3( 256 ), 0, stream,
			args.C + b0 * args.BatchStrideC, args.Bias, args.M, args.N, args.Ldc, args.BatchStrideC );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

template<int BM, int BN, int WAVES_M, int WAVES_N, int AMODE, int BMODE>
static int launchTile( hipStream_t stream, CMatMulArgs& args, int batch, bool vec, const CSliceMeeting* fixedMeeting )
{
	args.TilesM = ceilDiv( args.M, BM );
	args.TilesN = ceilDiv( args.N, BN );
	args.TilesNMagic = divisionMagic( args.TilesN );
	args.WoMagic = divisionMagic( args.Wo );
	args.HoMagic = divisionMagic( args.Ho );
	{
		const long long cBytes = ( static_cast<long long>( args.M - 1 ) * args.Ldc + args.N ) * 4;
		args.CBytes = ( args.Ldc >= args.N && cBytes > 0 && cBytes < 0x7fffff00LL ) ? static_cast<unsigned>( cBytes ) : 0u;
	}
	const long long tiles = static_cast<long long>( args.TilesM ) * args.TilesN;
	if( tiles > 0x7fffffffLL ) {
		setLastError( "matrix product: too many tiles" );
		return NH_ERR_ARGUMENT;
	}
	// K slices: when the tiles alone leave most compute units with a few workgroups, K is cut into slices that meet in
	// scratch memory or, where that is not possible, in C through fp32 atomic adds. Eight workgroups fit a compute unit.
	// The slice count is picked by a small model of the launch, fitted to measurements of 3x3 convolutions and of matrix
	// products: with w workgroups in all, the fullest compute unit runs n = ceil( w / 256 ) of them side by side when they
	// all fit at once ( w <= 2048 ), each as long as its K steps plus about 8 steps for its prologue, epilogue and the
	// meeting, and the matrix pipe is busy n / ( n + 1.7 ) of the time with n wavefronts per SIMD to pick from; beyond
	// 2048 the compute units refill as workgroups end and the imbalance shrinks to about 0.6 of a workgroup.
	// Every slice keeps at least 8 K steps.
	// an empty reduction ( K == 0 ) still launches: one step of masked loads, C receives the free term or keeps its value
	const int totalSteps = args.K > 0 ? ceilDiv( args.K, NH_KSTEP ) : 1;
	int splits = 1;
	const long long blocks = tiles * batch;
	auto launchCost = [&]( int slices ) -> double {
		const double perUnit = static_cast<double>( blocks * slices ) / 256.0;
		const double length = static_cast<double>( ceilDiv( totalSteps, slices ) ) + 8.0;
		if( blocks * slices <= 2048 ) {
			const double sideBySide = ceil( perUnit );
			return sideBySide * length * ( sideBySide + 1.7 ) / sideBySide;
		}
		return ( perUnit + 0.6 ) * length * ( 8.0 + 1.7 ) / 8.0;
	};
	if( args.ManySlices != 0 ) {
		// a gradient by a filter: a few tiles, a reduction over every pixel of the batch, up to hundreds of slices
		const int most = totalSteps / 8 > 0 ? totalSteps / 8 : 1;
		double best = 0;
		for( int s = 1; s <= most && ( s == 1 || blocks * s <= 4096 ); ++s ) {
			const double cost = launchCost( s );
			if( s == 1 || cost < best ) {
				best = cost;
				splits = s;
			}
		}
	// ( with a residual only slices that meet in scratch memory will do, see below )
	} else if( blocks < 1024 && totalSteps >= 32 && ( args.Residual == nullptr || ( batch == 1 && AMODE != AM_ConvClasses && BM * BN == 4096 ) ) ) {
		double best = 0;
		for( int s = 1; s <= 8 && s <= totalSteps / 8; ++s ) {
			const double cost = launchCost( s );
			if( s == 1 || cost < best ) {
				best = cost;
				splits = s;
			}
		}
	}
	// two slices of an even number of steps: the two halves share a workgroup of 8 wavefronts instead (KGROUPS = 2)
	bool twoGroups = false;
	if constexpr( BM == 64 && BN == 64 && BMODE == BM_RowsK && ( AMODE == AM_Conv || AMODE == AM_ConvTaps || AMODE == AM_RowsK ) ) {
		if( vec && splits == 2 && totalSteps % 2 == 0 && batch == 1 && args.ManySlices == 0 ) {
			twoGroups = true;
			splits = 1;
		}
	}
	args.StepsPerSplit = ceilDiv( totalSteps, splits );
	args.SplitK = ceilDiv( totalSteps, args.StepsPerSplit );
	// Tail mode: more tiles than run at once, and the last round of them would leave most of the device idle. The tiles
	// of the whole rounds run as they are; the rest is cut into K slices that fill that last round. Priced in rounds of
	// whole tiles, from measurements of the 3x3 convolutions: a round filled to the fraction f takes 0.17 + 0.85 f of a
	// full one (fewer workgroups per compute unit run faster, but not in proportion), a workgroup costs about 4 K steps
	// beyond its own, and the preset of the tail rows about 2 K steps of a round.
	const int slots = 256 * 5; // planned as above: the five that saturate a compute unit, not the eight that fit
	long long gridX = tiles;
	int tailRow = 0;
	if( splits == 1 && !twoGroups && batch == 1 && AMODE != AM_ConvClasses && args.Residual == nullptr && tiles >= slots && totalSteps >= 16 ) {
		long long full = tiles / slots * slots;
		full -= full % args.TilesN; // whole rows of tiles: the preset below covers the rows behind them
		const long long rest = tiles - full;
		auto roundsFor = []( double fill ) {
			const double whole = floor( fill );
			const double part = fill - whole;
			return whole + ( part > 0 ? 0.17 + 0.85 * part : 0.0 );
		};
		int best = 1;
		double bestCost = 0, unsplitCost = 0;
		for( int slices = 1; slices <= 8 && slices <= totalSteps / 8; ++slices ) {
			const double length = ( static_cast<double>( totalSteps ) / slices + 4.0 ) / ( totalSteps + 4.0 );
			const double cost = roundsFor( static_cast<double>( rest * slices ) / slots ) * length
				+ ( slices > 1 ? 2.0 / totalSteps : 0.0 );
			if( slices == 1 ) {
				unsplitCost = cost;
			}
			if( slices == 1 || cost < bestCost ) {
				bestCost = cost;
				best = slices;
			}
		}
		if( bestCost > unsplitCost - 0.03 ) {
			best = 1; // not worth the atomics
		}
		if( rest > 0 && best > 1 ) {
			args.FullTiles = static_cast<int>( full );
			args.TailTiles = static_cast<int>( rest );
			args.TailSteps = ceilDiv( totalSteps, best );
			args.TailSplit = ceilDiv( totalSteps, args.TailSteps );
			gridX = full + rest * args.TailSplit;
			tailRow = static_cast<int>( full / args.TilesN ) * BM;
		}
	}
	// Few slices per tile, one matrix: the slices meet through partial tiles in scratch memory and the last one to arrive
	// runs the epilogue, so there is no preset of C, no atomic add and no separate activation pass, and the sum has a
	// fixed order. (Not for the gradient by a filter with its dozens of slices, nor for the per-class launches, whose
	// slices may have nothing to do and would never arrive.) Falls back to atomics when the scratch cannot be had.
	if( ( args.SplitK > 1 || args.FullTiles > 0 ) && batch == 1 && args.ManySlices == 0 && AMODE != AM_ConvClasses
		&& BM * BN == 4096 )
	{
		const size_t slicedTiles = args.FullTiles > 0 ? args.TailTiles : static_cast<size_t>( tiles );
		const size_t slices = args.FullTiles > 0 ? args.TailSplit : args.SplitK;
		CSliceScratch scratch;
		if( fixedMeeting != nullptr ) {
			// the caller's place: no allocation, no look at the stream; the contents are whatever the last call left
			if( slicedTiles * slices * 4096 > fixedMeeting->PartialFloats || slicedTiles > fixedMeeting->CounterCount ) {
				setLastError( "the K slices of this launch need %zu bytes of partial tiles and %zu counters; the fixed scratch holds "
					"%zu bytes and %zu counters", slicedTiles * slices * 4096 * sizeof( float ), slicedTiles,
					fixedMeeting->PartialFloats * sizeof( float ), fixedMeeting->CounterCount );
				return NH_ERR_ARGUMENT;
			}
			hipLaunchKernelGGL( clearCountersKernel, dim3( ceilDiv( static_cast<long long>( slicedTiles ), 1024 ) ), dim3( 256 ), 0, stream,
				fixedMeeting->Counters, static_cast<int>( slicedTiles ) );
			args.Partials = fixedMeeting->Partials;
			args.Counters = fixedMeeting->Counters;
		} else if( sliceScratch( stream, slicedTiles * slices * 4096, slicedTiles, scratch ) ) {
			args.Partials = scratch.Partials;
			args.Counters = scratch.Counters;
		}
	}
	const bool meetInScratch = args.Partials != nullptr;
	if( args.Residual != nullptr && args.SplitK > 1 && !meetInScratch ) {
		// The residual is added by the one workgroup that writes a tile, which is the last slice to arrive at the meeting;
		// slices that add onto C with atomics have no such workgroup. No scratch ( a capturing stream ): one slice.
		args.StepsPerSplit = totalSteps;
		args.SplitK = 1;
	}
	// the rows of the tail tiles as a matrix product of their own: what the preset and the activation pass cover
	CMatMulArgs tail = args;
	tail.C += static_cast<long long>( tailRow ) * args.Ldc;
	tail.M = args.M - tailRow;
	if( args.FullTiles > 0 && !args.Accumulate && !meetInScratch ) {
		const int rc = presetResult( stream, tail, 1 );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	if( args.SplitK > 1 && !args.Accumulate && !meetInScratch ) {
		CMatMulArgs dense = args;
		if( AMODE == AM_ConvClasses ) {
			dense.M = args.DenseM; // the classes interleave in one dense result
		}
		const int rc = presetResult( stream, dense, AMODE == AM_ConvClasses ? 1 : batch );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	const CFusedActivation actAfter = args.Act;
	if( args.SplitK > 1 && !meetInScratch ) {
		args.Act.Type = NH_ACT_NONE;
	}
	// blockIdx.y is limited to 65535: walk larger batches in slices
	for( int b0 = 0; b0 < batch; b0 += 65535 ) {
		const int nb = batch - b0 < 65535 ? batch - b0 : 65535;
		CMatMulArgs a = args;
		a.A += b0 * args.BatchStrideA;
		a.B += b0 * args.BatchStrideB;
		a.C += b0 * args.BatchStrideC;
		const dim3 grid( static_cast<unsigned>( gridX ), nb, args.SplitK );
		if( twoGroups ) {
			if constexpr( BM == 64 && BN == 64 && BMODE == BM_RowsK && ( AMODE == AM_Conv || AMODE == AM_ConvTaps || AMODE == AM_RowsK ) ) {
				hipLaunchKernelGGL( ( matMulKernel<BM, BN, WAVES_M, WAVES_N, AMODE, BMODE, true, 2> ), grid, dim3( Threads * 2 ), 0, stream, a );
			}
		} else if( vec ) {
			hipLaunchKernelGGL( ( matMulKernel<BM, BN, WAVES_M, WAVES_N, AMODE, BMODE, true> ), grid, dim3( Threads ), 0, stream, a );
		} else if constexpr( AMODE != AM_ConvTaps ) {
			hipLaunchKernelGGL( ( matMulKernel<BM, BN, WAVES_M, WAVES_N, AMODE, BMODE, false> ), grid, dim3( Threads ), 0, stream, a );
		}
		if( args.FullTiles > 0 && actAfter.Type != NH_ACT_NONE && !meetInScratch ) {
			const long long total = static_cast<long long>( tail.M ) * args.N;
			const long long blocksAct = ( total + 1023 ) / 1024;
			hipLaunchKernelGGL( activateResultKernel, dim3( static_cast<unsigned>( blocksAct > 4096 ? 4096 : blocksAct ), 1 ), dim3( 256 ), 0,
				stream, tail.C, tail.M, args.N, args.Ldc, args.BatchStrideC, actAfter );
		}
		if( args.SplitK > 1 && actAfter.Type != NH_ACT_NONE && !meetInScratch ) {
			const long long total = static_cast<long long>( args.M ) * args.N;
			const long long blocksAct = ( total + 1023 ) / 1024;
			hipLaunchKernelGGL( activateResultKernel, dim3( static_cast<unsigned>( blocksAct > 4096 ? 4096 : blocksAct ), nb ), dim3( 256 ), 0,
				stream, a.C, args.M, args.N, args.Ldc, args.BatchStrideC, actAfter );
		}
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// Picks the workgroup tile. Measured on MI355X (convolutions of 64..512 channels, GEMMs up to 8192^3): the 64x64 tile
// wins or ties everywhere, because it puts the most workgroups on every compute unit (eight fit by LDS and registers; a 128x64 tile, five per compute unit with two
// accumulators per wavefront, is 0-25 % slower on the shapes of the benchmarks and 2 % faster only on 256 -> 256 channels
// over 65 536 pixels),
// and latency hiding across workgroups matters more at fp32 MFMA rates than the smaller tile's extra L2 traffic.
// Narrow outputs (N <= 32, and 96 or 160 columns) use 128x32 so that no MFMA block multiplies padding.
template<int AMODE, int BMODE>
static int launchMatMul( hipStream_t stream, CMatMulArgs& args, int batch, bool vec, const CSliceMeeting* fixedMeeting = nullptr )
{
	// ( 96 or 160 columns: three or five tiles of 32 columns instead of two or three of 64 the last of which is half padding;
	// 25088 x 96 x 384 30.4 -> 26.0 us, 6272 x 160 x 576 21.8 -> 17.3, 6272 x 160 x 960 28.5 -> 24.2 )
	if( args.N > 32 && !( args.N <= 160 && args.N % 64 == 32 ) ) {
		return launchTile<64, 64, 2, 2, AMODE, BMODE>( stream, args, batch, vec, fixedMeeting );
	}
	return launchTile<128, 32, 4, 1, AMODE, BMODE>( stream, args, batch, vec, fixedMeeting );
}

// The vector path addresses each operand with 32-bit byte offsets below BufferBytes.
static bool fitsBuffer( long long rows, long long pitch, long long width )
{
	return rows <= 0 || ( ( rows - 1 ) * pitch + width ) * 4 < static_cast<long long>( BufferBytes );
}

// ---------------------------------------------------------------------------------------------------------
// Short reductions over many rows: C[M x N] = act( A[M x K] * W[N x K]^T + bias ) (+ residual), K = 8 * KC <= 192,
// N <= 32 * NB, all dense. These are the pointwise convolutions of a depthwise-separable network at high resolution
// (16 -> 96, 24 -> 144, 144 -> 24 channels over 10^5..10^6 pixels): they move 4 ( K + N ) bytes per row for 2 K N
// flops, which at fp32 MFMA rates puts the matrix pipe at 25-50 % of its peak while the memory runs at full rate, so
// the two must overlap. The tiled kernel above, built around a long K loop, spends its time in prologues and
// epilogues and re-reads A once per 64 output columns.
// Here a wavefront owns 32 whole rows: it fetches them straight into MFMA operand registers (every lane its row's
// K values, 16 bytes per load: together the loads of a wavefront cover one contiguous piece of A), keeps them for
// all output columns, and walks the columns in blocks of 32 with W and the bias read from LDS, where the workgroup
// put them once. No barrier after that; wavefronts take further row blocks grid-stride.
// A wavefront's loads and stores complete in issue order, and the wait in front of a use counts the operations issued
// after the awaited one, so that count must be known when the kernel is compiled: every memory operation of the row-block
// loop is unconditional (raw buffer accesses; rows beyond M and columns beyond N get an out-of-range offset, which
// reads zeros and drops stores), the column blocks are unrolled (NB), and nothing but A, the residual and C touches
// memory inside the loop. The registers of A are refilled with the next row block's values right behind the last
// MFMAs that read them, the residual of a column block is requested one block ahead: in the steady state no
// wavefront waits for its own stores.
// MFMA e of the c-th group of 8 k reduces over { 8c + e, 8c + 4 + e } on both operands.
__device__ __forceinline__ float hSwishOf( float v )
{
	const float mid = v * ( v + 3.f ) * ( 1.f / 6.f );
	return v <= -3.f ? 0.f : ( v >= 3.f ? v : mid );
}

//
// The same kernel is the first layer of an image network ( RP > 0 ): a convolution over an image with one or three
// channels, whose reduction is short ( 3 x 3 x 3 = 27, 7 x 7 x 3 = 147 ) and whose result is many times larger than its
// input. A row of A is then the window of one output pixel: Fh runs of RowK = Fw * Cin consecutive floats of a
// channels-last image, laid out as Fh rows of RP = RowK rounded up to a multiple of 4 ( k = r * RP + j ). A lane's 16
// bytes of chunk c are four consecutive j of one filter row r, both known at compile time per half-wavefront, fetched
// with one 128-bit load at 4-byte alignment. What such a load brings along beyond the run ( j >= RowK: the next
// pixels ), before the image row's first element ( padding on the left: the row above ) or behind its last one is
// replaced by zeros when the registers are first used; filter rows above and below the image get an out-of-range offset;
// the descriptor ends with the image blob, and a 128-bit load is range-checked per component, so nothing is read
// beyond it. Offsets cannot be negative: the few pixels of the first image whose window begins in front of the blob
// ( top left corner, padding on the left ) lie in the first row blocks, which are the ones the prologue fetches, and
// those it fetches element by element.
struct CRowRuns {
	int H, W, Cin, Ho, Wo, Fh, RowK;
	int PadH, PadW, StrideH, StrideW;
	unsigned ABytes; // size of the image blob
	int SlowRows; // output pixels below this index: fetched element by element ( all of them in prologue blocks )
};

// where a lane's output pixel sits in the image
struct CRunState {
	int PixBytes; // byte offset of filter row 0, j = 0 ( negative where that lies in front of the blob )
	int Hi0; // image row of filter row 0
	int Lb, Span; // j is inside the image row and the run for Lb <= j < Lb + Span
};

// ( W is the MFMA's first operand and A its second: the 32 x 32 block comes out transposed, lane ( l32, half ) holding
// row l32 and, in registers 4g..4g+3, its columns 8g + 4 half .. + 3. The accumulator starts as the bias of those columns. )
template<int KC, int NB, bool RES, int RP>
__global__ __launch_bounds__( Threads, 2 )
void shortReductionKernel( const float* A, const float* W, const float* bias, float* C, int M, int N, int rowBlocks,
	const CFusedActivation actAsGiven, const float* residual, const CRowRuns geo )
{
	const CFusedActivation act = withParam( actAsGiven );
	constexpr int K = KC * 8;
	constexpr int Pitch = K + 4;
	constexpr int PatchPitch = 36;
	constexpr int RP_OR_ONE = RP > 0 ? RP : 1;
	constexpr int KR = RP > 0 ? ( K + RP - 1 ) / RP : 1; // filter rows that K spans ( those beyond Fh only round K up )
	// Column blocks worked on together, each with its own accumulator. The window loader's long reductions are bound by
	// the matrix pipe, and the two wavefronts per SIMD that registers and LDS leave room for keep it only half busy with
	// one chain of dependent MFMAs each; two independent chains per wavefront do what four wavefronts would.
	constexpr int Together = ( RP > 0 && NB % 2 == 0 ) ? 2 : 1;
	static_assert( !RES || Together == 1, "the residual is requested one column block ahead" );
	// ... and the chunks of a long reduction alternate between two chains per column block, added up at the end
	// ( measured: no gain on any shape once two column blocks run together; kept for single column blocks of the window loader )
	constexpr int Chains = ( RP > 0 && Together == 1 ) ? 2 : 1;
	// [32 * NB][Pitch], rows beyond N are zero; the bias, [32 * NB]; then one [32][36] output patch per wavefront
	extern __shared__ __attribute__( ( aligned( 16 ) ) ) float wLds[];
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int l32 = lane & 31;
	const int half = lane >> 5;

	float* biasLds = wLds + NB * 32 * Pitch;
	float* patch = biasLds + NB * 32 + wave * 32 * PatchPitch;
	const __amdgpu_buffer_rsrc_t bufA = RP > 0 ? __builtin_amdgcn_make_buffer_rsrc( const_cast<float*>( A ), 0, geo.ABytes, 0x00020000 )
		: makeBuffer( A );
	// C and the residual end where the matrix ends: rows beyond M are out of range by themselves
	const unsigned cBytes = static_cast<unsigned>( M ) * static_cast<unsigned>( N ) * 4u;
	const __amdgpu_buffer_rsrc_t bufC = __builtin_amdgcn_make_buffer_rsrc( C, 0, cBytes, 0x00020000 );
	const __amdgpu_buffer_rsrc_t bufR = __builtin_amdgcn_make_buffer_rsrc( const_cast<float*>( RES ? residual : C ), 0, cBytes, 0x00020000 );
	const unsigned rowBytes = static_cast<unsigned>( N ) * 4u;
	// a lane stores 16 bytes: columns col4..col4+3 of row q * 8 + lane / 8 of the 32 x 32 block, q = 0..3
	const int col4 = ( lane & 7 ) * 4;
	const unsigned laneOut = static_cast<unsigned>( lane >> 3 ) * rowBytes + col4 * 4u;
	const int stride = gridDim.x * 4;
	const float reluTop = act.Param > 0.f ? act.Param : __builtin_inff(); // the upper threshold of ReLU, if any

	auto rowOffset = [&]( int block ) -> unsigned {
		const int m = block * 32 + l32;
		return ( block < rowBlocks && m < M ) ? static_cast<unsigned>( m ) * ( K * 4u ) + half * 16u : OutOfRange;
	};
	auto outOffset = [&]( int block, int nb ) -> unsigned {
		// ( blocks beyond the last one start beyond cBytes )
		return nb * 32 + col4 < N ? static_cast<unsigned>( block ) * 32u * rowBytes + nb * 128u + laneOut : OutOfRange;
	};

	// the pixel of this lane in row block `block` ( RP > 0 )
	const int rowBytesIn = RP > 0 ? geo.W * geo.Cin * 4 : 0;
	auto locate = [&]( int block ) -> CRunState {
		CRunState s = { 0, -0x40000000, 0, 0 }; // no filter row meets the image: every chunk out of range
		const int m = block * 32 + l32;
		if( block < rowBlocks && m < M ) {
			const int wo = m % geo.Wo;
			const int t = m / geo.Wo;
			const int ho = t % geo.Ho;
			const int n = t / geo.Ho;
			const int wc0 = ( wo * geo.StrideW - geo.PadW ) * geo.Cin;
			s.Hi0 = ho * geo.StrideH - geo.PadH;
			s.PixBytes = ( n * geo.H + s.Hi0 ) * rowBytesIn + wc0 * 4;
			s.Lb = wc0 < 0 ? -wc0 : 0;
			const int inRow = geo.W * geo.Cin - wc0;
			const int ub = geo.RowK < inRow ? geo.RowK : inRow;
			s.Span = ub > s.Lb ? ub - s.Lb : 0;
		}
		return s;
	};
	// filter row and position in it of this lane's piece of chunk c
	auto chunkRow = [&]( int c ) -> int { return half != 0 ? ( 8 * c + 4 ) / RP_OR_ONE : ( 8 * c ) / RP_OR_ONE; };
	auto chunkPos = [&]( int c ) -> int { return half != 0 ? ( 8 * c + 4 ) % RP_OR_ONE : ( 8 * c ) % RP_OR_ONE; };
	auto chunkOffset = [&]( const CRunState& s, int c ) -> unsigned {
		const int r = chunkRow( c );
		const bool meets = static_cast<unsigned>( s.Hi0 + r ) < static_cast<unsigned>( geo.H ) && r < geo.Fh;
		return meets ? static_cast<unsigned>( s.PixBytes + r * rowBytesIn + chunkPos( c ) * 4 ) : OutOfRange;
	};
	// zeros behind the run's end, for lanes whose window lies inside the image row ( j < RowK is all that can fail, and
	// only in the last positions of a filter row )
	auto maskRunEnd = [&]( int c, float4 v ) -> float4 {
		const int j0 = ( 8 * c ) % RP_OR_ONE;
		const int j1 = ( 8 * c + 4 ) % RP_OR_ONE;
		if( j0 + 3 >= RP_OR_ONE - 3 || j1 + 3 >= RP_OR_ONE - 3 ) {
			const int j = half != 0 ? j1 : j0;
			v.x = j < geo.RowK ? v.x : 0.f;
			v.y = j + 1 < geo.RowK ? v.y : 0.f;
			v.z = j + 2 < geo.RowK ? v.z : 0.f;
			v.w = j + 3 < geo.RowK ? v.w : 0.f;
		}
		return v;
	};
	auto maskChunk = [&]( const CRunState& s, int c, float4 v ) -> float4 {
		const unsigned t = static_cast<unsigned>( chunkPos( c ) - s.Lb );
		const unsigned span = static_cast<unsigned>( s.Span );
		v.x = t < span ? v.x : 0.f;
		v.y = t + 1u < span ? v.y : 0.f;
		v.z = t + 2u < span ? v.z : 0.f;
		v.w = t + 3u < span ? v.w : 0.f;
		return v;
	};

	if( RP > 0 ) {
		// the filter [N][Fh][RowK] into rows of Fh x RP ( + what rounds K up ), zeros in the padding
#pragma unroll 8
		for( int idx = tid; idx < NB * 32 * K; idx += Threads ) {
			const int n = idx / K;
			const int k = idx - n * K;
			const int r = k / RP_OR_ONE;
			const int j = k - r * RP_OR_ONE;
			wLds[n * Pitch + k] = ( n < N && r < geo.Fh && j < geo.RowK ) ? W[( static_cast<long long>( n ) * geo.Fh + r ) * geo.RowK + j] : 0.f;
		}
	} else {
		for( int idx = tid; idx < NB * 32 * ( K / 4 ); idx += Threads ) {
			const int n = idx / ( K / 4 );
			const int k4 = idx - n * ( K / 4 );
			const float4 v = n < N ? *reinterpret_cast<const float4*>( W + static_cast<long long>( n ) * K + k4 * 4 )
				: make_float4( 0.f, 0.f, 0.f, 0.f );
			*reinterpret_cast<float4*>( wLds + n * Pitch + k4 * 4 ) = v;
		}
	}
	for( int n = tid; n < NB * 32; n += Threads ) {
		biasLds[n] = ( bias != nullptr && n < N ) ? bias[n] : 0.f;
	}
	__syncthreads();

	int block = blockIdx.x * 4 + wave;
	float4 a[KC];
	CRunState cur = { 0, 0, 0, 0 };
	if( RP > 0 ) {
		cur = locate( block );
		if( block * 32 < geo.SlowRows ) {
			// a block with pixels whose window begins in front of the blob: element by element, nothing out of bounds
			const long long pixFloats = cur.PixBytes / 4; // ( exact: a multiple of 4, also when negative )
#pragma unroll
			for( int c = 0; c < KC; ++c ) {
				const int r = chunkRow( c );
				const int j0 = chunkPos( c );
				const bool meets = static_cast<unsigned>( cur.Hi0 + r ) < static_cast<unsigned>( geo.H ) && r < geo.Fh;
				const float* from = A + ( pixFloats + static_cast<long long>( r ) * ( rowBytesIn / 4 ) + j0 );
				float e[4];
#pragma unroll
				for( int i = 0; i < 4; ++i ) {
					const bool inside = meets && static_cast<unsigned>( j0 + i - cur.Lb ) < static_cast<unsigned>( cur.Span );
					e[i] = inside ? from[i] : 0.f;
				}
				a[c] = make_float4( e[0], e[1], e[2], e[3] );
			}
		} else {
#pragma unroll
			for( int c = 0; c < KC; ++c ) {
				a[c] = bufferLoad4( bufA, chunkOffset( cur, c ) );
			}
		}
	} else {
		const unsigned first = rowOffset( block );
#pragma unroll
		for( int c = 0; c < KC; ++c ) {
			a[c] = bufferLoad4( bufA, first + c * 32u ); // an out-of-range row reads zeros
		}
	}

	float4 res[4];
	{
		if( RES ) {
			const unsigned o = outOffset( block, 0 );
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				res[q] = bufferLoad4( bufR, o + q * 8u * rowBytes );
			}
		}
		// Stores that go nowhere, as many as a pass over the last column blocks issues: the loop is entered with the same sequence of outstanding operations that its
		// own last column block leaves behind, so the compiler's wait counts for the first MFMAs skip the stores.
#pragma unroll
		for( int q = 0; q < 4 * Together; ++q ) {
			bufferStore4( bufC, OutOfRange + q * 16u, make_float4( 0.f, 0.f, 0.f, 0.f ) );
		}
	}
	for( ; block < rowBlocks; block += stride ) {
		const unsigned nextRows = RP > 0 ? 0u : rowOffset( block + stride );
		// RP > 0: what the loads for the next row block need, per filter row: its byte offset at j = 0, out of range
		// where the row lies above or below the image
		CRunState next = { 0, 0, 0, 0 };
		unsigned nextRow[KR];
		if( RP > 0 ) {
			next = locate( block + stride );
#pragma unroll
			for( int r = 0; r < KR; ++r ) {
				const bool meets = static_cast<unsigned>( next.Hi0 + r ) < static_cast<unsigned>( geo.H ) && r < geo.Fh;
				nextRow[r] = meets ? static_cast<unsigned>( next.PixBytes + r * rowBytesIn ) : OutOfRange;
			}
		}
		// every lane's window inside its image row ( wave-uniform ): only the run's end needs zeros then
		// ( the other wavefronts, those with a pixel at the left or right border or behind the last one, first put zeros
		// wherever a lane's bounds ask for them; the registers are changed in place, under a branch without MFMAs )
		const bool plain = RP > 0 && __builtin_amdgcn_ballot_w64( cur.Lb != 0 || cur.Span != geo.RowK ) == 0;
		if( RP > 0 && !plain ) {
#pragma unroll
			for( int c = 0; c < KC; ++c ) {
				a[c] = maskChunk( cur, c, a[c] );
			}
		}
#pragma unroll
		for( int nb = 0; nb < NB; nb += Together ) {
			const bool lastColumns = nb + Together >= NB; // known when the loop is unrolled
			f32x16 accs[Together * Chains];
#pragma unroll
			for( int t = 0; t < Together; ++t ) {
				const float* b = biasLds + ( nb + t ) * 32 + half * 4;
#pragma unroll
				for( int g = 0; g < 4; ++g ) {
					const float4 v = *reinterpret_cast<const float4*>( b + g * 8 );
					accs[t][g * 4] = v.x;
					accs[t][g * 4 + 1] = v.y;
					accs[t][g * 4 + 2] = v.z;
					accs[t][g * 4 + 3] = v.w;
				}
				if constexpr( Chains > 1 ) {
#pragma unroll
					for( int i = 0; i < 16; ++i ) {
						accs[Together + t][i] = 0.f;
					}
				}
			}
			const float* wRow = wLds + ( nb * 32 + l32 ) * Pitch + half * 4;
			float4 resNext[4];
			float* mine = patch + l32 * PatchPitch + half * 4;
			// The MFMAs of the column blocks, and the first block's move to the LDS patch: nothing else stands between the
			// MFMAs and the first use of their result, in one basic block. Masks: 0 none, 1 the run's end.
			auto pass = [&]( auto masks ) {
				constexpr int Masks = decltype( masks )::value;
#pragma unroll
				for( int c = 0; c < KC; ++c ) {
					float4 w[Together];
#pragma unroll
					for( int t = 0; t < Together; ++t ) {
						w[t] = *reinterpret_cast<const float4*>( wRow + t * 32 * Pitch + c * 8 );
					}
					if( Masks == 1 ) {
						a[c] = maskRunEnd( c, a[c] ); // first use of what the loads brought
					}
					// ( the later column block first: its chain is the older one when the blocks go out in ascending order )
#pragma unroll
					for( int t = Together - 1; t >= 0; --t ) {
						f32x16& chain = accs[( c % Chains ) * Together + t];
						chain = __builtin_amdgcn_mfma_f32_32x32x2f32( w[t].x, a[c].x, chain, 0, 0, 0 );
					}
#pragma unroll
					for( int t = Together - 1; t >= 0; --t ) {
						f32x16& chain = accs[( c % Chains ) * Together + t];
						chain = __builtin_amdgcn_mfma_f32_32x32x2f32( w[t].y, a[c].y, chain, 0, 0, 0 );
					}
#pragma unroll
					for( int t = Together - 1; t >= 0; --t ) {
						f32x16& chain = accs[( c % Chains ) * Together + t];
						chain = __builtin_amdgcn_mfma_f32_32x32x2f32( w[t].z, a[c].z, chain, 0, 0, 0 );
					}
#pragma unroll
					for( int t = Together - 1; t >= 0; --t ) {
						f32x16& chain = accs[( c % Chains ) * Together + t];
						chain = __builtin_amdgcn_mfma_f32_32x32x2f32( w[t].w, a[c].w, chain, 0, 0, 0 );
					}
					if( lastColumns ) {
						if( RP > 0 ) {
							const unsigned o0 = nextRow[( 8 * c ) / RP_OR_ONE] + ( ( 8 * c ) % RP_OR_ONE ) * 4u;
							const unsigned o1 = nextRow[( 8 * c + 4 ) / RP_OR_ONE] + ( ( 8 * c + 4 ) % RP_OR_ONE ) * 4u;
							a[c] = bufferLoad4( bufA, half != 0 ? o1 : o0 );
							// ( left to itself the scheduler gathers these loads behind the last MFMA, and the next row
							// block begins by waiting for them )
							__builtin_amdgcn_sched_barrier( 0 );
						} else {
							a[c] = bufferLoad4( bufA, nextRows + c * 32u );
						}
					}
				}
				// the residual of the column block that follows ( of the next row block behind the last one )
				if( RES ) {
					const unsigned o = lastColumns ? outOffset( block + stride, 0 ) : outOffset( block, nb + 1 );
#pragma unroll
					for( int q = 0; q < 4; ++q ) {
						resNext[q] = bufferLoad4( bufR, o + q * 8u * rowBytes );
					}
				}
				f32x16 acc = accs[0];
				if constexpr( Chains > 1 ) {
#pragma unroll
					for( int i = 0; i < 16; ++i ) {
						acc[i] += accs[Together][i];
					}
				}
#pragma unroll
				for( int g = 0; g < 4; ++g ) {
					*reinterpret_cast<float4*>( mine + g * 8 ) = make_float4( acc[g * 4], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3] );
				}
			};
			if( RP > 0 && nb == 0 ) {
				pass( std::integral_constant<int, 1>() );
			} else {
				pass( std::integral_constant<int, 0>() );
			}
			// The block goes out through a wavefront-private patch of LDS in which the lanes regroup: a lane then holds
			// four neighbouring columns of a row such that one store instruction covers whole 128-byte runs of 8 rows
			// ( stored as they come out of the MFMA, an instruction would touch 32 rows with 32 bytes each ). The
			// activation, with its branches on the type, is applied to what comes back from the patch.
#pragma unroll
			for( int t = 0; t < Together; ++t ) {
				if( t > 0 ) {
					// ( a later block of the group: its MFMAs were issued before the first block's last ones )
					f32x16 acc = accs[t];
					if constexpr( Chains > 1 ) {
#pragma unroll
						for( int i = 0; i < 16; ++i ) {
							acc[i] += accs[Together + t][i];
						}
					}
#pragma unroll
					for( int g = 0; g < 4; ++g ) {
						*reinterpret_cast<float4*>( mine + g * 8 ) = make_float4( acc[g * 4], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3] );
					}
				}
				// ( same wavefront: the LDS unit executes its reads after its writes, no barrier needed )
				float4 v[4];
#pragma unroll
				for( int q = 0; q < 4; ++q ) {
					v[q] = *reinterpret_cast<const float4*>( patch + ( q * 8 + ( lane >> 3 ) ) * PatchPitch + col4 );
				}
				if( act.Type == NH_ACT_RELU ) {
#pragma unroll
					for( int q = 0; q < 4; ++q ) {
						// NaN becomes 0, as in VectorReLU: the maximum of a NaN and a number is the number
						v[q].x = __builtin_fminf( __builtin_fmaxf( v[q].x, 0.f ), reluTop );
						v[q].y = __builtin_fminf( __builtin_fmaxf( v[q].y, 0.f ), reluTop );
						v[q].z = __builtin_fminf( __builtin_fmaxf( v[q].z, 0.f ), reluTop );
						v[q].w = __builtin_fminf( __builtin_fmaxf( v[q].w, 0.f ), reluTop );
					}
				} else if( act.Type == NH_ACT_HSWISH ) {
#pragma unroll
					for( int q = 0; q < 4; ++q ) {
						v[q].x = hSwishOf( v[q].x );
						v[q].y = hSwishOf( v[q].y );
						v[q].z = hSwishOf( v[q].z );
						v[q].w = hSwishOf( v[q].w );
					}
				}
				const unsigned o = outOffset( block, nb + t );
#pragma unroll
				for( int q = 0; q < 4; ++q ) {
					if( RES ) {
						v[q].x += res[q].x;
						v[q].y += res[q].y;
						v[q].z += res[q].z;
						v[q].w += res[q].w;
					}
					bufferStore4( bufC, o + q * 8u * rowBytes, v[q] );
				}
			}
			if( RES ) {
#pragma unroll
				for( int q = 0; q < 4; ++q ) {
					res[q] = resNext[q];
				}
			}
		}
		cur = next;
	}
}

static constexpr size_t shortReductionLds( int K, int nb )
{
	return ( static_cast<size_t>( nb ) * 32 * ( K + 4 ) + nb * 32 + 4 * 32 * 36 ) * sizeof( float );
}

// ( false, and nothing launched: a window loader whose element-wise blocks would not all be first blocks )
template<int KC, int NB, bool RES, int RP = 0>
static bool launchShortReduction( hipStream_t stream, const float* a, const float* w, const float* bias, float* c, int M, int N,
	const CFusedActivation& act, const float* residual, const CRowRuns& geo = CRowRuns() )
{
	const int rowBlocks = ceilDiv( M, 32 );
	const int groups = ceilDiv( rowBlocks, 4 );
	const size_t lds = shortReductionLds( KC * 8, NB );
	// The wavefronts walk the row blocks grid-stride. Narrow outputs ( one block of columns: read-bound, a long prologue
	// that copies W to LDS ): the grid is what the device holds at once ( registers and LDS decide, both depend on KC and
	// NB ), so that no second, partly filled round of workgroups trails behind the first. Wide outputs ( write-bound ):
	// four rounds' worth of workgroups, which drift apart instead of loading and storing in step with each other
	// ( 16 -> 96 channels over 1.6 M pixels: 144 -> 133 us ).
	static std::mutex lock;
	static std::map<int, int> residentFor;
	int resident = 0;
	{
		int device = 0;
		( void )hipGetDevice( &device );
		std::lock_guard<std::mutex> guard( lock );
		int& known = residentFor[device];
		if( known == 0 ) {
			int perUnit = 0, units = 0;
			if( hipOccupancyMaxActiveBlocksPerMultiprocessor( &perUnit, shortReductionKernel<KC, NB, RES, RP>, Threads, lds ) != hipSuccess
				|| hipDeviceGetAttribute( &units, hipDeviceAttributeMultiprocessorCount, device ) != hipSuccess
				|| perUnit <= 0 || units <= 0 )
			{
				( void )hipGetLastError();
				perUnit = 2;
				units = 256;
			}
			known = perUnit * units;
		}
		resident = known;
	}
	if( NB > 1 && RP == 0 ) {
		resident *= 4; // ( the window loader's reductions are long enough to be bound by the matrix pipe: one round )
	}
	const int grid = groups < resident ? groups : resident;
	if( RP > 0 && geo.SlowRows > grid * 128 ) {
		return false;
	}
	hipLaunchKernelGGL( ( shortReductionKernel<KC, NB, RES, RP> ), dim3( grid ), dim3( Threads ), lds, stream,
		a, w, bias, c, M, N, rowBlocks, act, residual, geo );
	return true;
}

// One kernel per count of column blocks that 64 KB of LDS hold next to the output patches.
template<int KC, int NB>
static bool launchShortReductionColumns( hipStream_t stream, const float* a, const float* w, const float* bias, float* c, int M, int N,
	const CFusedActivation& act, const float* residual )
{
	if constexpr( NB >= 1 && shortReductionLds( KC * 8, NB >= 1 ? NB : 1 ) <= 64 * 1024 ) {
		if( ceilDiv( N, 32 ) == NB ) {
			if( residual != nullptr ) {
				return launchShortReduction<KC, NB, true>( stream, a, w, bias, c, M, N, act, residual );
			}
			return launchShortReduction<KC, NB, false>( stream, a, w, bias, c, M, N, act, residual );
		}
		return launchShortReductionColumns<KC, NB - 1>( stream, a, w, bias, c, M, N, act, residual );
	} else if constexpr( NB >= 1 ) {
		return launchShortReductionColumns<KC, NB - 1>( stream, a, w, bias, c, M, N, act, residual );
	} else {
		return false;
	}
}

// true (and launched) when the product has the shape this kernel is for
static bool tryShortReduction( hipStream_t stream, const float* a, int lda, const float* w, int ldb, float* c, int ldc,
	int M, int N, int K, const float* bias, const CFusedActivation& act, const float* residual, int* rc )
{
	if( lda != K || ldb != K || ldc != N || M < 16384 || K % 8 != 0 || K > 192 || N > 192 || N % 4 != 0
		|| !isAligned16( a ) || !isAligned16( w ) || !isAligned16( c ) || !isAligned16( residual )
		|| !fitsBuffer( M, K, K ) || !fitsBuffer( M + 32, N, N ) )
	{
		return false;
	}
	bool launched = false;
	switch( K / 8 ) {
		case 2: launched = launchShortReductionColumns<2, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 3: launched = launchShortReductionColumns<3, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 4: launched = launchShortReductionColumns<4, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 6: launched = launchShortReductionColumns<6, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 8: launched = launchShortReductionColumns<8, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 12: launched = launchShortReductionColumns<12, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 18: launched = launchShortReductionColumns<18, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		case 24: launched = launchShortReductionColumns<24, 6>( stream, a, w, bias, c, M, N, act, residual ); break;
		default: break;
	}
	if( !launched ) {
		return false;
	}
	const hipError_t err = hipGetLastError();
	if( err != hipSuccess ) {
		setLastError( "short-reduction product: launch failed: %s", hipGetErrorString( err ) );
		*rc = NH_ERR_HIP;
	} else {
		*rc = NH_OK;
	}
	return true;
}

// ---- plain products with long reductions and large results -------------------------------------------------------
// C[M x N] (+)= act( A[M x K] * B[N x K]^T + bias ) (+ residual), both operands K-major: the products of fully connected
// layers over thousands of rows ( transformer feed-forward 8192 x 2048 x 512 and 8192 x 512 x 2048, the input product of
// an LSTM layer 8192 x 1024 x 256 ).
// Workgroup tile 128 x 128, K step 16, two LDS buffers of [row][16 + 4], in two shapes:
//   eight wavefronts ( 2 x 4 ), each 64 rows x 32 columns = two 32 x 32 MFMA blocks that share their B operand; three
//   workgroups fit a compute unit;
//   four wavefronts ( 2 x 2 ), each 64 x 64 = four blocks; four workgroups fit a compute unit.
// Against the 64 x 64 tile of matMulKernel every value that reaches LDS feeds twice as many MFMAs and every fragment
// read 1.5 to 2 times as many, which on this part shows as a higher sustained clock as much as in fewer stalls, and
// eight waves per workgroup keep two to six waves on every SIMD even when the tiles only just cover the compute units.
// Measured against the 64 x 64 tile ( us ): 8192 x 512 x 2048 129 -> 123, 8192 x 512 x 512 39 -> 35, 8192 x 1024 x 256
// 40 -> 36.5, 8192 x 2048 x 2048 550 -> 469 ( 146.5 TFLOP/s ) with eight wavefronts. With 1024 tiles and a reduction of 32
// steps ( 8192 x 2048 x 512 ) the eight-wave shape runs 768 workgroups at once and the remaining 256 afterwards on a
// device that is three quarters idle: 130 to 150 us, depending on how far the first ones had drifted apart; four
// workgroups of four waves per compute unit hold all 1024 at once: 130 us.
// Each thread fetches 128-bit pieces of A and B ( raw buffer loads: rows beyond the matrix read as zeros ) into SETS
// register sets; with one set the values wait a whole step before they go to LDS, which is enough while several
// workgroups share a compute unit; two sets pay where a compute unit holds one workgroup.
struct CLongProductArgs {
	const float* A;
	const float* B;
	float* C;
	const float* Bias;     // per column, may be null
	const float* Residual; // C's layout, may be null, may be C
	int M, N, K;
	int Lda, Ldb, Ldc;
	long long BatchStrideA, BatchStrideB, BatchStrideC;
	int TilesN;
	int Accumulate;
	CFusedActivation Act;
};

constexpr int LongTile = 128;

// WGM x WGN wavefronts, each MI x NI blocks of 32 x 32; WPE: wavefronts per SIMD the registers must leave room for
// RAGGED: K is not a multiple of the step
template<int WGM, int WGN, int MI, int NI, int SETS, int WPE, bool RAGGED>
__global__ __launch_bounds__( 64 * WGM * WGN, WPE )
void longProductKernel( const CLongProductArgs args )
{
	constexpr int KS = NH_KSTEP, LdsK = KS + 4, KQ = KS / 4;
	constexpr int T = 64 * WGM * WGN;
	constexpr int BM = 32 * WGM * MI, BN = 32 * WGN * NI;
	constexpr int ASlots = BM * KQ / T, BSlots = BN * KQ / T;
	static_assert( KS == 16 && BM * KQ % T == 0 && BN * KQ % T == 0, "whole load slots per thread" );
	__shared__ __attribute__( ( aligned( 16 ) ) ) float lds[2][( BM + BN ) * LdsK];

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int waveM = wave / WGN, waveN = wave % WGN;
	const int l32 = lane & 31, half = lane >> 5;

	const int tile = xcdSwizzle( blockIdx.x, gridDim.x );
	const int m0 = ( tile / args.TilesN ) * BM;
	const int n0 = ( tile % args.TilesN ) * BN;
	const int batch = blockIdx.y;
	const int M = args.M, N = args.N, K = args.K;
	const float* baseA = args.A + batch * args.BatchStrideA;
	const float* baseB = args.B + batch * args.BatchStrideB;

	// load slots of this thread: tile row ( dealt so that the two rows eight neighbouring lanes store to LDS are four
	// apart: conflict-free at a pitch of 20 floats ) and 128-bit column
	const int kq = ( tid & 3 ) * 4;
	auto rowOfSlot = [&]( int i ) -> int {
		const int q = ( tid + i * T ) >> 2;
		return ( q & ~7 ) | ( ( q & 1 ) << 2 ) | ( ( q & 6 ) >> 1 );
	};
	unsigned offA[ASlots], offB[BSlots];
#pragma unroll
	for( int i = 0; i < ASlots; ++i ) {
		const int m = m0 + rowOfSlot( i );
		offA[i] = m < M ? static_cast<unsigned>( m * args.Lda + kq ) * 4u : OutOfRange;
	}
#pragma unroll
	for( int i = 0; i < BSlots; ++i ) {
		const int n = n0 + rowOfSlot( i );
		offB[i] = n < N ? static_cast<unsigned>( n * args.Ldb + kq ) * 4u : OutOfRange;
	}
	const int kSteps = ( K + KS - 1 ) / KS;
	const bool inLastStep = ( kSteps - 1 ) * KS + kq < K; // RAGGED: the last step has columns beyond K, they must read as zeros

	float4 rA[SETS][ASlots], rB[SETS][BSlots];
	// Every step of the reduction, the last ones included, runs the same code with the same number of loads in flight
	// ( the waits in front of the LDS stores count them ): a step behind the last one is requested through a descriptor of
	// size zero, which answers with zeros without touching memory and costs two scalar instructions. No vector
	// instruction: a wave's vector instructions wait for its MFMAs in flight, and two selects per step on the lanes'
	// offsets cost 3 % ( 8192 x 2048 x 2048: 469 -> 484 us ). Only a K that ends inside a step ( RAGGED, a kernel of its
	// own ) pays them, for the per-lane mask of its last step.
	auto load = [&]( int step, int set ) {
		const unsigned uni = static_cast<unsigned>( step ) * ( KS * 4u );
		const unsigned range = step < kSteps ? BufferBytes : 0u;
		const __amdgpu_buffer_rsrc_t bufA = __builtin_amdgcn_make_buffer_rsrc( const_cast<float*>( baseA ), 0, range, 0x00020000 );
		const __amdgpu_buffer_rsrc_t bufB = __builtin_amdgcn_make_buffer_rsrc( const_cast<float*>( baseB ), 0, range, 0x00020000 );
		const bool masked = RAGGED && step == kSteps - 1 && !inLastStep;
#pragma unroll
		for( int i = 0; i < ASlots; ++i ) {
			rA[set][i] = bufferLoad4( bufA, masked ? OutOfRange : offA[i], uni );
		}
#pragma unroll
		for( int i = 0; i < BSlots; ++i ) {
			rB[set][i] = bufferLoad4( bufB, masked ? OutOfRange : offB[i], uni );
		}
	};
	auto store = [&]( int buf, int set ) {
#pragma unroll
		for( int i = 0; i < ASlots; ++i ) {
			*reinterpret_cast<float4*>( &lds[buf][rowOfSlot( i ) * LdsK + kq] ) = rA[set][i];
		}
#pragma unroll
		for( int i = 0; i < BSlots; ++i ) {
			*reinterpret_cast<float4*>( &lds[buf][( BM + rowOfSlot( i ) ) * LdsK + kq] ) = rB[set][i];
		}
	};

	f32x16 acc[MI][NI];
#pragma unroll
	for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
		for( int ni = 0; ni < NI; ++ni ) {
#pragma unroll
			for( int r = 0; r < 16; ++r ) {
				acc[mi][ni][r] = 0.f;
			}
		}
	}
	// fragments of one group of 8 k: lane ( l32, half ) holds k = 8 g + 4 half .. + 3 of its row, MFMA j reduces over
	// { 8 g + j, 8 g + 4 + j } on both operands
	struct CFrag {
		float A[MI][4];
		float B[NI][4];
	};
	CFrag frag[2];
	const int fragA = ( waveM * 32 * MI + l32 ) * LdsK + half * 4;
	const int fragB = ( BM + waveN * 32 * NI + l32 ) * LdsK + half * 4;
	auto readFrag = [&]( int buf, int g, CFrag& f ) {
#pragma unroll
		for( int mi = 0; mi < MI; ++mi ) {
			const float4 v = *reinterpret_cast<const float4*>( &lds[buf][fragA + mi * 32 * LdsK + g * 8] );
			f.A[mi][0] = v.x; f.A[mi][1] = v.y; f.A[mi][2] = v.z; f.A[mi][3] = v.w;
		}
#pragma unroll
		for( int ni = 0; ni < NI; ++ni ) {
			const float4 v = *reinterpret_cast<const float4*>( &lds[buf][fragB + ni * 32 * LdsK + g * 8] );
			f.B[ni][0] = v.x; f.B[ni][1] = v.y; f.B[ni][2] = v.z; f.B[ni][3] = v.w;
		}
	};
	auto multiply = [&]( const CFrag& f ) {
#pragma unroll
		for( int j = 0; j < 4; ++j ) {
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
				for( int ni = 0; ni < NI; ++ni ) {
					acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32( f.A[mi][j], f.B[ni][j], acc[mi][ni], 0, 0, 0 );
				}
			}
		}
	};

	// Step ks multiplies out of LDS buffer ks % 2 while the operands of step ks + 1 go from registers to the other buffer
	// and those of step ks + 1 + SETS are requested. The one barrier of a step sits between its two groups of 8 k: the
	// second group's fragments were fetched ahead of it, so behind it nobody reads the buffer any more ( it is the one
	// the next step stores to ), and the first fragments of the next step are fetched right behind it.
	constexpr int Ahead = SETS + 1;
	auto step = [&]( int ks, auto parity ) {
		constexpr int nxt = decltype( parity )::value; // == ( ks + 1 ) % 2
		constexpr int cur = nxt ^ 1;
		constexpr int set = SETS == 2 ? nxt : 0;
		store( nxt, set ); // ( behind the last step: zeros that nobody multiplies )
		load( ks + Ahead, set );
		__builtin_amdgcn_sched_barrier( 0 );
		readFrag( cur, 1, frag[1] );
		__builtin_amdgcn_sched_barrier( 0 );
		multiply( frag[0] );
		__builtin_amdgcn_sched_barrier( 0 );
		__syncthreads();
		readFrag( nxt, 0, frag[0] );
		__builtin_amdgcn_sched_barrier( 0 );
		multiply( frag[1] );
		__builtin_amdgcn_sched_barrier( 0 );
	};

	load( 0, 0 );
	store( 0, 0 );
	if( SETS == 2 ) {
		load( 1, 1 );
		load( 2, 0 );
	} else {
		load( 1, 0 );
	}
	__syncthreads();
	readFrag( 0, 0, frag[0] );
	int ks = 0;
	for( ; ks + 1 < kSteps; ks += 2 ) {
		step( ks, std::integral_constant<int, 1>() );
		step( ks + 1, std::integral_constant<int, 0>() );
	}
	if( ks < kSteps ) {
		step( ks, std::integral_constant<int, 1>() );
	}

	// lane ( l32, half ) holds, of each block, one column of rows ( r / 4 ) * 8 + half * 4 + r % 4
	float* C = args.C + batch * args.BatchStrideC;
	const float* residual = args.Residual != nullptr ? args.Residual + batch * args.BatchStrideC : nullptr;
	const float actParam = withParam( args.Act ).Param; // ( the threshold may live in device memory )
			const float reluTop = actParam > 0.f ? actParam : __builtin_inff();
	const bool accumulate = args.Accumulate != 0;
	const int rowBase = m0 + waveM * 32 * MI + half * 4;
	// what is the same for the whole tile is decided once, here, and not per element: 32 or 64 elements per lane and up
	// to six wavefronts per SIMD make an epilogue with a handful of branches per element cost microseconds
	auto write = [&]( auto typeOf, auto extraOf, auto checkedOf ) {
		constexpr int Type = decltype( typeOf )::value;
		constexpr bool Extra = decltype( extraOf )::value;     // accumulate and / or residual
		constexpr bool Checked = decltype( checkedOf )::value; // the tile hangs over the last row
#pragma unroll
		for( int ni = 0; ni < NI; ++ni ) {
			const int n = n0 + waveN * 32 * NI + ni * 32 + l32;
			if( n >= N ) {
				continue;
			}
			const float bias = args.Bias != nullptr ? args.Bias[n] : 0.f;
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					const int m = rowBase + mi * 32 + ( r >> 2 ) * 8 + ( r & 3 );
					if( !Checked || m < M ) {
						const long long at = static_cast<long long>( m ) * args.Ldc + n;
						float v = acc[mi][ni][r] + bias;
						if constexpr( Extra ) {
							if( accumulate ) {
								v += C[at];
							}
						}
						v = applyActivationOf<Type>( v, reluTop );
						if constexpr( Extra ) {
							if( residual != nullptr ) {
								v += residual[at];
							}
						}
						C[at] = v;
					}
				}
			}
		}
	};
	auto writeAs = [&]( auto typeOf ) {
		if( accumulate || residual != nullptr ) {
			write( typeOf, std::true_type(), std::true_type() );
		} else if( m0 + BM > M ) {
			write( typeOf, std::false_type(), std::true_type() );
		} else {
			write( typeOf, std::false_type(), std::false_type() );
		}
	};
	if( args.Act.Type == NH_ACT_RELU ) {
		writeAs( std::integral_constant<int, NH_ACT_RELU>() );
	} else if( args.Act.Type == NH_ACT_HSWISH ) {
		writeAs( std::integral_constant<int, NH_ACT_HSWISH>() );
	} else {
		writeAs( std::integral_constant<int, NH_ACT_NONE>() );
	}
}

// true ( and launched ) when the product is one this kernel is for: vector loads possible, a reduction of at least eight
// steps, and enough 128 x 128 tiles to give every compute unit the same number of workgroups to within a quarter ( results
// with fewer tiles, or tiles that would be mostly padding, stay with the 64 x 64 tiles and their K slices )
static bool tryLongProduct( hipStream_t stream, const CMatMulArgs& a, int batch, bool vec, int* rc )
{
	if( !vec || a.K < 8 * NH_KSTEP || a.M < LongTile || a.N < LongTile / 2 || batch > 65535 ) {
		return false;
	}
	const long long tilesM = ceilDiv( a.M, LongTile ), tilesN = ceilDiv( a.N, LongTile );
	const long long tiles = tilesM * tilesN * batch;
	if( tilesM * tilesN > 0x7fffffffLL ) {
		return false;
	}
	const double covered = static_cast<double>( a.M ) * a.N / ( static_cast<double>( tilesM * LongTile ) * ( tilesN * LongTile ) );
	const long long unitsAtOnce = 256;
	const long long deepest = ( tiles + unitsAtOnce - 1 ) / unitsAtOnce;
	const double balance = static_cast<double>( tiles ) / static_cast<double>( deepest * unitsAtOnce );
	if( covered < 0.85 || ( tiles < 3 * unitsAtOnce && balance < 0.75 ) ) {
		return false;
	}
	CLongProductArgs args = {};
	args.A = a.A; args.B = a.B; args.C = a.C; args.Bias = a.Bias; args.Residual = a.Residual;
	args.M = a.M; args.N = a.N; args.K = a.K;
	args.Lda = a.Lda; args.Ldb = a.Ldb; args.Ldc = a.Ldc;
	args.BatchStrideA = a.BatchStrideA; args.BatchStrideB = a.BatchStrideB; args.BatchStrideC = a.BatchStrideC;
	args.TilesN = static_cast<int>( tilesN );
	args.Accumulate = a.Accumulate;
	args.Act = a.Act;
	const dim3 grid( static_cast<unsigned>( tilesM * tilesN ), batch );
	const int kSteps = ceilDiv( a.K, NH_KSTEP );
	auto launch = [&]( auto ragged ) {
		constexpr bool Ragged = decltype( ragged )::value;
		if( tiles <= unitsAtOnce ) {
			// one workgroup per compute unit: two waves per SIMD, the operands get two steps to arrive
			hipLaunchKernelGGL( ( longProductKernel<2, 4, 2, 1, 2, 4, Ragged> ), grid, dim3( 512 ), 0, stream, args );
		} else if( tiles > 3 * unitsAtOnce && tiles <= 4 * unitsAtOnce && kSteps <= 64 ) {
			// more than the three workgroups of eight waves that fit a compute unit, and a reduction too short for them
			// to drift apart: four workgroups of four waves hold all the tiles at once
			hipLaunchKernelGGL( ( longProductKernel<2, 2, 2, 2, 1, 4, Ragged> ), grid, dim3( 256 ), 0, stream, args );
		} else {
			hipLaunchKernelGGL( ( longProductKernel<2, 4, 2, 1, 1, 6, Ragged> ), grid, dim3( 512 ), 0, stream, args );
		}
	};
	if( a.K % NH_KSTEP != 0 ) {
		launch( std::true_type() );
	} else {
		launch( std::false_type() );
	}
	const hipError_t err = hipGetLastError();
	if( err != hipSuccess ) {
		setLastError( "long product: launch failed: %s", hipGetErrorString( err ) );
		*rc = NH_ERR_HIP;
	} else {
		*rc = NH_OK;
	}
	return true;
}

// C = A * B^T (+ bias) with row strides; also the inner product of the convolution with a 1x1 filter.
int matMulNTFused( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate, const CFusedActivation& act, const float* residual );

int matMulNT( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate )
{
	const CFusedActivation none = { NH_ACT_NONE, 0.f };
	return matMulNTFused( stream, a, lda, b, ldb, c, ldc, M, N, K, batch, strideA, strideB, strideC, bias, accumulate, none, nullptr );
}

static int matMulNTMeeting( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate, const CFusedActivation& act, const float* residual, const CSliceMeeting* fixedMeeting );

// ... and C = act( A * B^T + bias ) + residual, the epilogue of the fused blocks
int matMulNTFused( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate, const CFusedActivation& act, const float* residual )
{
	return matMulNTMeeting( stream, a, lda, b, ldb, c, ldc, M, N, K, batch, strideA, strideB, strideC, bias, accumulate, act,
		residual, nullptr );
}

static int matMulNTMeeting( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate, const CFusedActivation& act, const float* residual, const CSliceMeeting* fixedMeeting )
{
	if( M == 0 || N == 0 || batch == 0 ) {
		return NH_OK;
	}
	CMatMulArgs args = {};
	args.A = a; args.B = b; args.C = c; args.Bias = bias;
	args.M = M; args.N = N; args.K = K;
	args.Lda = lda; args.Ldb = ldb; args.Ldc = ldc;
	args.BatchStrideA = strideA; args.BatchStrideB = strideB; args.BatchStrideC = strideC;
	args.Accumulate = accumulate ? 1 : 0;
	args.Act = act;
	args.Residual = residual;
	int rc = NH_OK;
	if( batch == 1 && !accumulate && tryShortReduction( stream, a, lda, b, ldb, c, ldc, M, N, K, bias, act, residual, &rc ) ) {
		return rc;
	}
	const bool vec = isAligned16( a ) && isAligned16( b ) && K % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0
		&& strideA % 4 == 0 && strideB % 4 == 0 && fitsBuffer( M, lda, K ) && fitsBuffer( N, ldb, K );
	if( fixedMeeting == nullptr && tryLongProduct( stream, args, batch, vec, &rc ) ) {
		return rc;
	}
	return launchMatMul<AM_RowsK, BM_RowsK>( stream, args, batch, vec, fixedMeeting );
}

// ---- batched products of small matrices -----------------------------------------------------------------------
// C[b] = A[b] ( M x K ) * B[b] ( K x N ), all row-major, for batches of products that are too small to hide memory
// latency one 64 x 64 tile and one 16-k step at a time ( the two products of an attention head: 256 x 64 by 64 x 256,
// 256 x 256 by 256 x 64 ). A workgroup owns a strip of rows of one product and walks over all of its tiles: a step is
// ( 64 columns, KS k ) with k running fastest, the operands of step s + 2 are on their way from memory while those of
// step s + 1 sit in registers and those of step s are multiplied out of LDS, and the accumulators are written whenever a
// tile's last k chunk is done. One launch = as many workgroups as there are 64-row strips, all resident together.
// MI: 32-row blocks per wavefront ( the strip has 64 MI rows; two blocks are two independent chains of MFMAs per wave ),
// KS: k values per step.
template<int MI, int KS>
__global__ __launch_bounds__( Threads, 2 )
void batchedStripKernel( const float* A, const float* B, float* C, int M, int N, int K, int lda, int ldb, int ldc,
	long long strideA, long long strideB, long long strideC, int tilesM, int tilesN, int kChunks, const float* scale )
{
	// ( a factor for every element of the result, read from device memory: the VectorMultiply of a CLinearLayer behind the
	// product, done on the accumulators' way out; the accumulator is the value that call would have read, so the bits are its )
	const float alpha = scale != nullptr ? *scale : 1.f;
	constexpr int BM = 64 * MI;
	constexpr int PitchA = KS + 4, PitchB = 68;
	constexpr int QA = KS / 4;                 // float4 columns of an A tile row
	constexpr int RowsA = Threads / QA;        // A tile rows fetched by one pass of the workgroup
	constexpr int SlotsA = BM / RowsA, SlotsB = KS / 16;
	__shared__ __attribute__( ( aligned( 16 ) ) ) float lds[2][BM * PitchA + KS * PitchB]; // [buffer]{ A [m][k], B [k][n] }
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int waveM = wave >> 1, waveN = wave & 1;
	const int l32 = lane & 31, half = lane >> 5;
	const int id = xcdSwizzle( blockIdx.x, gridDim.x ); // the strips of one product share its B: same XCD, same L2
	const int batch = id / tilesM;
	const int m0 = ( id % tilesM ) * BM;
	const __amdgpu_buffer_rsrc_t bufA = makeBuffer( A + batch * strideA );
	const __amdgpu_buffer_rsrc_t bufB = makeBuffer( B + batch * strideB );
	C += batch * strideC;

	const int qA = ( tid % QA ) * 4, rA0 = tid / QA;
	const int qB = ( tid & 15 ) * 4, rB0 = tid >> 4;
	unsigned rowA[SlotsA];
#pragma unroll
	for( int i = 0; i < SlotsA; ++i ) {
		const int m = m0 + rA0 + RowsA * i;
		rowA[i] = m < M ? static_cast<unsigned>( m * lda + qA ) * 4u : OutOfRange;
	}
	float4 rA[SlotsA], rB[SlotsB];
	auto loadTiles = [&]( int step ) {
		const int kBase = ( step % kChunks ) * KS;
		const int n = ( step / kChunks ) * 64 + qB;
		const bool kOkA = kBase + qA < K; // K % 4 == 0: a float4 along k lies inside or outside
#pragma unroll
		for( int i = 0; i < SlotsA; ++i ) {
			// a valid offset is below 2 GiB, so adding to an out-of-range one stays out of range
			rA[i] = bufferLoad4( bufA, kOkA ? rowA[i] + static_cast<unsigned>( kBase ) * 4u : OutOfRange );
		}
#pragma unroll
		for( int i = 0; i < SlotsB; ++i ) {
			const int k = kBase + rB0 + 16 * i;
			rB[i] = bufferLoad4( bufB, k < K && n < N ? static_cast<unsigned>( k * ldb + n ) * 4u : OutOfRange );
		}
	};
	auto storeTiles = [&]( int buf ) {
#pragma unroll
		for( int i = 0; i < SlotsA; ++i ) {
			*reinterpret_cast<float4*>( &lds[buf][( rA0 + RowsA * i ) * PitchA + qA] ) = rA[i];
		}
#pragma unroll
		for( int i = 0; i < SlotsB; ++i ) {
			*reinterpret_cast<float4*>( &lds[buf][BM * PitchA + ( rB0 + 16 * i ) * PitchB + qB] ) = rB[i];
		}
	};
	f32x16 acc[MI];
#pragma unroll
	for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
		for( int r = 0; r < 16; ++r ) {
			acc[mi][r] = 0.f;
		}
	}
	const int steps = tilesN * kChunks;
	loadTiles( 0 );
	storeTiles( 0 );
	if( steps > 1 ) {
		loadTiles( 1 );
	}
	__syncthreads();
	for( int step = 0; step < steps; ++step ) {
		const int cur = step & 1;
		// buffer cur ^ 1 was read in step - 1, and every wave has passed the barrier that closed it
		if( step + 1 < steps ) {
			storeTiles( cur ^ 1 );
		}
		if( step + 2 < steps ) {
			loadTiles( step + 2 );
		}
		__builtin_amdgcn_sched_barrier( 0 );
		const float* tA = &lds[cur][( waveM * 32 * MI + l32 ) * PitchA + half * 4];
		const float* tB = &lds[cur][BM * PitchA + ( half * 4 ) * PitchB + waveN * 32 + l32];
#pragma unroll
		for( int g = 0; g < KS / 8; ++g ) {
			// lane ( row or column l32, half ) holds k = 8 g + 4 half + j for MFMA j: the same permutation of k on both operands
			float4 a[MI];
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
				a[mi] = *reinterpret_cast<const float4*>( tA + mi * 32 * PitchA + g * 8 );
			}
			float b[4];
#pragma unroll
			for( int j = 0; j < 4; ++j ) {
				b[j] = tB[( g * 8 + j ) * PitchB];
			}
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
				acc[mi] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[mi].x, b[0], acc[mi], 0, 0, 0 );
			}
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
				acc[mi] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[mi].y, b[1], acc[mi], 0, 0, 0 );
			}
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
				acc[mi] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[mi].z, b[2], acc[mi], 0, 0, 0 );
			}
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
				acc[mi] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[mi].w, b[3], acc[mi], 0, 0, 0 );
			}
		}
		if( ( step + 1 ) % kChunks == 0 ) {
			const int n = ( step / kChunks ) * 64 + waveN * 32 + l32;
#pragma unroll
			for( int mi = 0; mi < MI; ++mi ) {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					const int m = m0 + waveM * 32 * MI + mi * 32 + ( r >> 2 ) * 8 + half * 4 + ( r & 3 );
					if( m < M && n < N ) {
						C[static_cast<long long>( m ) * ldc + n] = acc[mi][r] * alpha;
					}
					acc[mi][r] = 0.f;
				}
			}
		}
		__syncthreads();
	}
}

// Whether a batched row-major product goes to batchedStripKernel: vector loads possible, many strips, and a reduction of
// at most 256 ( longer ones keep the general kernel busy long enough per tile ).
static bool tryBatchedStrips( hipStream_t stream, const CMatMulArgs& args, int batch, bool vec, const float* scale )
{
	if( !vec || batch < 2 || args.Accumulate || args.K <= 0 || args.K > 256 ) {
		return false;
	}
	// measured on the two products of an attention head ( 256 products of 256 x 64 by 64 x 256 and of 256 x 256 by 256 x 64 ):
	// 64-row strips with 32-k steps 27.5 / 24.6 us, with 64-k steps 29.7 / 27.7, 128-row strips ( two chains of MFMAs per
	// wave ) with 32-k steps 28.7 / 25.1; the general kernel 35.2 / 27.0
	constexpr int KS = 32;
	const int tilesM = ceilDiv( args.M, 64 );
	const long long groups = static_cast<long long>( tilesM ) * batch;
	if( groups < 512 || groups > 0x7fffffffLL ) {
		return false;
	}
	hipLaunchKernelGGL( ( batchedStripKernel<1, KS> ), dim3( static_cast<unsigned>( groups ) ), dim3( Threads ), 0, stream,
		args.A, args.B, args.C, args.M, args.N, args.K, args.Lda, args.Ldb, args.Ldc,
		args.BatchStrideA, args.BatchStrideB, args.BatchStrideC, tilesM, ceilDiv( args.N, 64 ), ceilDiv( args.K, KS ), scale );
	return true;
}

// C = A * B, A is M x K, B is K x N, all row-major.
// scale: a device scalar that every element of the result is to be multiplied by, if the kernel that takes the product can
// do that on the way out ( *scaled says whether it did; the caller multiplies behind the product otherwise )
int matMulNN( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC, bool accumulate,
	const float* scale, bool* scaled )
{
	if( scaled != nullptr ) {
		*scaled = false;
	}
	if( M == 0 || N == 0 || batch == 0 ) {
		return NH_OK;
	}
	CMatMulArgs args = {};
	args.A = a; args.B = b; args.C = c; args.Bias = nullptr;
	args.M = M; args.N = N; args.K = K;
	args.Lda = lda; args.Ldb = ldb; args.Ldc = ldc;
	args.BatchStrideA = strideA; args.BatchStrideB = strideB; args.BatchStrideC = strideC;
	args.Accumulate = accumulate ? 1 : 0;
	const bool vec = isAligned16( a ) && isAligned16( b ) && K % 4 == 0 && N % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0
		&& strideA % 4 == 0 && strideB % 4 == 0 && fitsBuffer( M, lda, K ) && fitsBuffer( K, ldb, N );
	if( tryBatchedStrips( stream, args, batch, vec, scaled != nullptr ? scale : nullptr ) ) {
		if( scaled != nullptr ) {
			*scaled = scale != nullptr;
		}
		NH_LAUNCH_CHECK();
		return NH_OK;
	}
	return launchMatMul<AM_RowsK, BM_RowsN>( stream, args, batch, vec );
}

// C (+)= A^T * B, A is K x M (stored), B is K x N, all row-major; the reduction runs over the stored rows.
int matMulTN( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC, bool accumulate )
{
	if( M == 0 || N == 0 || batch == 0 ) {
		return NH_OK;
	}
	CMatMulArgs args = {};
	args.A = a; args.B = b; args.C = c; args.Bias = nullptr;
	args.M = M; args.N = N; args.K = K;
	args.Lda = lda; args.Ldb = ldb; args.Ldc = ldc;
	args.BatchStrideA = strideA; args.BatchStrideB = strideB; args.BatchStrideC = strideC;
	args.Accumulate = accumulate ? 1 : 0;
	const bool vec = isAligned16( a ) && isAligned16( b ) && M % 4 == 0 && N % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0
		&& strideA % 4 == 0 && strideB % 4 == 0 && fitsBuffer( K, lda, M ) && fitsBuffer( K, ldb, N );
	return launchMatMul<AM_RowsM, BM_RowsN>( stream, args, batch, vec );
}

// The first layer of an image network through the short-reduction kernel's window loader: true (and launched) for the
// filter shapes it is built for.
template<int KC, int RP>
static bool launchWindowReduction( hipStream_t stream, const float* a, const float* w, const float* bias, float* c, int M, int N,
	const CFusedActivation& act, const CRowRuns& geo )
{
	if( N <= 32 ) {
		return launchShortReduction<KC, 1, false, RP>( stream, a, w, bias, c, M, N, act, nullptr, geo );
	}
	return launchShortReduction<KC, 2, false, RP>( stream, a, w, bias, c, M, N, act, nullptr, geo );
}

static bool tryWindowReduction( hipStream_t stream, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act, int* rc )
{
	const long long m = static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth;
	const long long imageFloats = static_cast<long long>( d.batch ) * d.height * d.width * d.channels;
	const int rowK = d.filterWidth * d.channels;
	const int rowPitch = ( rowK + 3 ) / 4 * 4;
	if( d.dilationHeight != 1 || d.dilationWidth != 1 || m < 16384 || d.filterCount > 64 || d.filterCount % 4 != 0
		|| !isAligned16( result ) || imageFloats * 4 >= static_cast<long long>( BufferBytes )
		|| !fitsBuffer( m + 32, d.filterCount, d.filterCount ) )
	{
		return false;
	}
	CRowRuns geo = {};
	geo.H = d.height; geo.W = d.width; geo.Cin = d.channels; geo.Ho = d.resultHeight; geo.Wo = d.resultWidth;
	geo.Fh = d.filterHeight; geo.RowK = rowK;
	geo.PadH = d.paddingHeight; geo.PadW = d.paddingWidth; geo.StrideH = d.strideHeight; geo.StrideW = d.strideWidth;
	geo.ABytes = static_cast<unsigned>( imageFloats * 4 );
	// windows that begin in front of the blob: first image, filter row on image row 0, padding on the left
	geo.SlowRows = d.paddingWidth > 0 ? ( d.paddingHeight / d.strideHeight + 1 ) * d.resultWidth : 0;
	const int M = static_cast<int>( m );
	const int N = d.filterCount;
	const int kc = ( d.filterHeight * rowPitch + 7 ) / 8;
	bool launched = false;
	if( rowPitch == 12 && kc == 5 ) { // 3 x 3 over RGB
		launched = launchWindowReduction<5, 12>( stream, source, filter, freeTerm, result, M, N, act, geo );
	} else if( rowPitch == 24 && kc == 21 ) { // 7 x 7 over RGB
		launched = launchWindowReduction<21, 24>( stream, source, filter, freeTerm, result, M, N, act, geo );
	} else if( rowPitch == 4 && kc == 2 ) { // 3 x 3 over one channel
		launched = launchWindowReduction<2, 4>( stream, source, filter, freeTerm, result, M, N, act, geo );
	}
	if( !launched ) {
		return false;
	}
	const hipError_t err = hipGetLastError();
	if( err != hipSuccess ) {
		setLastError( "window reduction: launch failed: %s", hipGetErrorString( err ) );
		*rc = NH_ERR_HIP;
	} else {
		*rc = NH_OK;
	}
	return true;
}

int convImplicitGemm( hipStream_t stream, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act, const CSliceMeeting* fixedMeeting = nullptr )
{
	CMatMulArgs args = {};
	args.Act = act;
	args.A = source; args.B = filter; args.C = result; args.Bias = freeTerm;
	const long long m = static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth;
	args.M = static_cast<int>( m );
	args.N = d.filterCount;
	args.K = d.filterHeight * d.filterWidth * d.channels;
	args.Lda = 0; args.Ldb = args.K; args.Ldc = d.filterCount;
	args.H = d.height; args.W = d.width; args.Cin = d.channels;
	args.Ho = d.resultHeight; args.Wo = d.resultWidth; args.Fh = d.filterHeight; args.Fw = d.filterWidth;
	args.PadH = d.paddingHeight; args.PadW = d.paddingWidth;
	args.StrideH = d.strideHeight; args.StrideW = d.strideWidth;
	args.DilH = d.dilationHeight; args.DilW = d.dilationWidth;
	if( args.M == 0 || args.N == 0 ) {
		return NH_OK;
	}
	const bool vec = isAligned16( source ) && isAligned16( filter ) && d.channels % 4 == 0
		&& fitsBuffer( 1, 0, static_cast<long long>( d.batch ) * d.height * d.width * d.channels )
		&& fitsBuffer( d.filterCount, args.K, args.K );
	if( d.filterHeight == 1 && d.filterWidth == 1 && d.strideHeight == 1 && d.strideWidth == 1
		&& d.paddingHeight == 0 && d.paddingWidth == 0 )
	{
		// a pointwise convolution over a channels-last image is the plain product image[M x Cin] * filter[Cout x Cin]^T
		return matMulNTMeeting( stream, source, d.channels, filter, d.channels, result, d.filterCount, args.M, args.N, d.channels,
			1, 0, 0, 0, freeTerm, false, act, nullptr, fixedMeeting );
	}
	if( d.filterHeight == 1 && d.filterWidth == 1 ) {
		return launchMatMul<AM_Conv1x1, BM_RowsK>( stream, args, 1, vec, fixedMeeting );
	}
	if( d.channels % 4 != 0 ) {
		int rc = NH_OK;
		if( tryWindowReduction( stream, d, source, filter, freeTerm, result, act, &rc ) ) {
			return rc;
		}
	}
	if( d.channels % 4 != 0 && d.dilationWidth == 1
		&& fitsBuffer( 1, 0, static_cast<long long>( d.batch ) * d.height * d.width * d.channels )
		&& fitsBuffer( d.filterCount, args.K, args.K ) )
	{
		args.RowK = d.filterWidth * d.channels;
		args.RowPitch = ( args.RowK + 3 ) / 4 * 4;
		args.AFloats = d.batch * d.height * d.width * d.channels;
		args.BFloats = d.filterCount * d.filterHeight * args.RowK;
		args.K = d.filterHeight * args.RowPitch; // reduction length as the kernel walks it; Ldb keeps the filter's own
		return launchMatMul<AM_ConvRows, BM_RowsK>( stream, args, 1, true, fixedMeeting );
	}
	if( vec && d.channels % NH_KSTEP == 0 ) {
		return launchMatMul<AM_ConvTaps, BM_RowsK>( stream, args, 1, true, fixedMeeting );
	}
	return launchMatMul<AM_Conv, BM_RowsK>( stream, args, 1, vec, fixedMeeting );
}

// ---- gradients of the convolution ------------------------------------------------------------------------------

// filter [Cout][taps][Cin] -> [Cin][taps][Cout]: the filter of the convolution that maps the output gradient back
__global__ __launch_bounds__( 256 ) void swapFilterChannelsKernel( const float* filter, float* swapped, int cout, int taps, int cin )
{
	const int total = cout * taps * cin;
	for( int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256 ) {
		const int co = i % cout;
		const int t = ( i / cout ) % taps;
		const int ci = i / ( cout * taps );
		swapped[i] = filter[( co * taps + t ) * cin + ci];
	}
}

// inputDiff[n,hi,wi,ci] = freeTerm[ci] + sum over ( kh, kw, co ) of outputDiff[n, (hi+p-kh*d)/s, (wi+p-kw*d)/s, co] *
// filter[co,kh,kw,ci], the terms whose divisions are exact and in range: the forward kernel on the output gradient as
// its image, with padding -p, dilation -d, the division by the stride, and the filter with its channel axes swapped.
// Which class a filter tap belongs to and where it goes inside the class's filter
struct CTapClasses {
	int StrideH, StrideW, DilH, DilW;
	int FirstH[2], FirstW[2];   // by residue: the first tap of the class along that axis
	int CountW[2];              // by residue: taps of the class along the width
	int K[MaxConvClasses];
	long long BOffset[MaxConvClasses];
};

// filter [Cout][Fh][Fw][Cin] -> per class [Cin][its taps][Cout]
__global__ __launch_bounds__( 256 ) void packClassFiltersKernel( const float* filter, float* packed, int cout, int fh, int fw,
	int cin, const CTapClasses t )
{
	const int total = cout * fh * fw * cin;
	for( int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256 ) {
		const int ci = i % cin;
		const int kw = ( i / cin ) % fw;
		const int kh = ( i / ( cin * fw ) ) % fh;
		const int co = i / ( cin * fw * fh );
		const int rh = ( kh * t.DilH ) % t.StrideH;
		const int rw = ( kw * t.DilW ) % t.StrideW;
		const int cls = rh * t.StrideW + rw;
		const int tap = ( kh - t.FirstH[rh] ) / t.StrideH * t.CountW[rw] + ( kw - t.FirstW[rw] ) / t.StrideW;
		packed[t.BOffset[cls] + static_cast<long long>( ci ) * t.K[cls] + tap * cout + co] = filter[i];
	}
}

static int gcd( int a, int b ) { return b == 0 ? a : gcd( b, a % b ); }

// The strided case of convBackwardData: true when it took the launch. A pixel hi of the input meets tap kh only when
// hi + pad - kh * dil is a multiple of the stride, so the pixels fall into stride^2 classes by ( hi + pad ) mod stride,
// each with its own subset of the taps; per class the sum is a stride-1 convolution without a single masked tap.
static bool convBackwardDataByClasses( hipStream_t stream, const nhConvDesc& d, const float* outputDiff, const float* filter,
	const float* freeTerm, float* inputDiff, float* packedFilter, int& rc )
{
	const int sh = d.strideHeight, sw = d.strideWidth;
	if( ( sh == 1 && sw == 1 ) || sh > 2 || sw > 2 || gcd( d.dilationHeight, sh ) != 1 || gcd( d.dilationWidth, sw ) != 1 ) {
		return false;
	}
	CMatMulArgs args = {};
	CTapClasses taps = {};
	taps.StrideH = sh; taps.StrideW = sw; taps.DilH = d.dilationHeight; taps.DilW = d.dilationWidth;
	// per axis and residue r: first pixel of the class, pixel count, first tap, tap count, source offset of pixel 0 / tap 0
	struct CAxis { int First, Count, FirstTap, Taps, Base; };
	auto axis = []( int size, int pad, int stride, int dil, int filterSize, int r ) {
		CAxis a = {};
		a.First = ( ( r - pad ) % stride + stride ) % stride;
		a.Count = a.First < size ? ( size - a.First + stride - 1 ) / stride : 0;
		a.FirstTap = 0;
		while( ( a.FirstTap * dil ) % stride != r ) {
			++a.FirstTap; // exists below stride: dil and stride are coprime
		}
		a.Taps = a.FirstTap < filterSize ? ( filterSize - a.FirstTap + stride - 1 ) / stride : 0;
		a.Base = ( a.First + pad - a.FirstTap * dil ) / stride; // exact
		return a;
	};
	long long offset = 0;
	int maxM = 0, maxK = 0;
	for( int rh = 0; rh < sh; ++rh ) {
		const CAxis h = axis( d.height, d.paddingHeight, sh, d.dilationHeight, d.filterHeight, rh );
		taps.FirstH[rh] = h.FirstTap;
		for( int rw = 0; rw < sw; ++rw ) {
			const CAxis w = axis( d.width, d.paddingWidth, sw, d.dilationWidth, d.filterWidth, rw );
			taps.FirstW[rw] = w.FirstTap;
			taps.CountW[rw] = w.Taps;
			CConvClass& c = args.Class[rh * sw + rw];
			c.Fh = h.Taps; c.Fw = w.Taps;
			c.K = h.Taps * w.Taps * d.filterCount;
			// source pixel of result pixel j through tap t: Base + j - t * dil
			c.PadH = -h.Base; c.PadW = -w.Base;
			c.Ho = h.Count; c.Wo = w.Count;
			c.M = d.batch * h.Count * w.Count;
			c.OutH0 = h.First; c.OutW0 = w.First;
			c.BOffset = offset;
			taps.K[rh * sw + rw] = c.K;
			taps.BOffset[rh * sw + rw] = offset;
			offset += static_cast<long long>( c.K ) * d.channels;
			maxM = c.M > maxM ? c.M : maxM;
			maxK = c.K > maxK ? c.K : maxK;
		}
	}
	const int filterSize = d.filterCount * d.filterHeight * d.filterWidth * d.channels;
	hipLaunchKernelGGL( packClassFiltersKernel, dim3( ceilDiv( filterSize, 1024 ) ), dim3( 256 ), 0, stream,
		filter, packedFilter, d.filterCount, d.filterHeight, d.filterWidth, d.channels, taps );
	// A filter narrower than the stride ( the 1 x 1 / 2 shortcut of a residual network ) leaves classes that no tap reaches:
	// their pixels are the free term or zero. One pass sets the whole result to that, and only the classes with taps are
	// multiplied ( as four classes the shortcut's 51 MB took 40 us, three quarters of it tiles that only wrote zeros ).
	int liveClasses = 0;
	bool idlePixels = false;
	maxM = 0; maxK = 0;
	for( int cls = 0; cls < sh * sw; ++cls ) {
		const CConvClass c = args.Class[cls];
		if( c.M == 0 ) {
			continue;
		}
		if( c.K == 0 ) {
			idlePixels = true;
			continue;
		}
		args.Class[liveClasses++] = c;
		maxM = c.M > maxM ? c.M : maxM;
		maxK = c.K > maxK ? c.K : maxK;
	}
	if( idlePixels ) {
		CMatMulArgs dense = {};
		dense.C = inputDiff; dense.Bias = freeTerm;
		dense.M = d.batch * d.height * d.width; dense.N = d.channels; dense.Ldc = d.channels;
		rc = presetResult( stream, dense, 1 );
		if( rc != NH_OK ) {
			return true;
		}
	}
	if( liveClasses == 0 ) {
		return true;
	}
	args.A = outputDiff; args.B = packedFilter; args.C = inputDiff; args.Bias = freeTerm;
	args.M = maxM; args.N = d.channels; args.K = maxK;
	args.Lda = 0; args.Ldb = maxK; args.Ldc = d.channels;
	args.H = d.resultHeight; args.W = d.resultWidth; args.Cin = d.filterCount;
	args.StrideH = 1; args.StrideW = 1;
	args.DilH = -d.dilationHeight; args.DilW = -d.dilationWidth;
	args.OutH = d.height; args.OutW = d.width; args.OutUpH = sh; args.OutUpW = sw;
	args.DenseM = d.batch * d.height * d.width;
	const bool vec = isAligned16( outputDiff ) && isAligned16( packedFilter ) && d.filterCount % 4 == 0
		&& fitsBuffer( 1, 0, static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth * d.filterCount )
		&& fitsBuffer( 1, 0, static_cast<long long>( filterSize ) );
	rc = launchMatMul<AM_ConvClasses, BM_RowsK>( stream, args, liveClasses, vec );
	return true;
}

// ---- input gradient of a 7 x 7 / 2 convolution from 3 to 64 channels ( the stem of the ImageNet networks ) -----------
// As a product per input pixel the result has 3 columns, and a matrix tile spends nine tenths of its work on padding
// ( 1.4 ms at 64 x 224 x 224 ). Turned round, every pixel of the output gradient is a row of 64 values times the
// filter as a 64 x 147 matrix, and the 147 products are the pixel's contributions to the 7 x 7 x 3 window of the input
// gradient it looks at: a product with hardly any padding, followed by sums over overlapping windows.
//
// A workgroup takes tiles of 16 x 16 output-gradient pixels, one after the other: 256 operand rows, two blocks of 32 per
// wave, a lane holding its pixel's 64 values in registers for the whole tile. The filter's columns ( column n = input
// channel x 49 + tap, 64 values each, transposed by a small launch in front ) are walked 32 at a time: per block of rows
// 32 v_mfma_f32_32x32x2 ( number j takes output channel 32 half + j from both operands, so a lane's values are adjacent
// in memory ), then every accumulator register is added to its place in the WAVE's own window in LDS; the place is the
// sum of a term of the row ( 8 per lane ) and a term of the column ( one per chunk ). The adds are plain LDS reads and
// writes ( LDS float atomics took six times as long ), which needs the places of one round to differ over the whole wave:
// two rows and two columns meet in one place only when 2 x + kx = 2 x' + kx' and 2 y + ky = 2 y' + ky', i.e. for pixels
// at most 3 apart in x and in y. So wave w takes the pixel rows y = w, w + 4, w + 8, w + 12, and accumulator register
// 4 q + i of a lane is pixel x = 4 X + i: register i of all eight groups ( 2 blocks x 4 ) and both half-waves are
// 16 pixels 4 apart in x or y, one round. Four rounds per chunk, each read - add - write; a wave's LDS operations complete
// in order. A wave's window is four bands of 7 rows x 37 x 3 values.
//
// The tile's 37 x 37 x 3 window ( the sum of the four waves' windows, in wave order ) overlaps its neighbours' by 5 pixels,
// so it goes to scratch memory, and a second launch adds up the at most four windows that cover an input pixel, in a
// fixed order, with the free term: no run differs from another.
constexpr int SgWindow = 37;                        // 2 x + kx for x < 16, kx < 7
constexpr int SgWindowFloats = SgWindow * SgWindow * 3;
constexpr int SgBandFloats = 7 * SgWindow * 3;      // one row of source pixels: 7 rows of the window
constexpr int SgWaveFloats = 4 * SgBandFloats;
constexpr int SgColumns = 147;                      // 3 channels x 49 taps
constexpr int SgStagePitch = 68;                    // floats per pixel where a row of pixels passes through LDS

constexpr int SgPackedFilterFloats = 5 * 8 * 64 * 4;

typedef float stemAcc __attribute__( ( ext_vector_type( 16 ) ) );

// filter [64][49][3] -> [chunk][i][lane][e]: output channel 32 half + 4 i + e of column 32 chunk + l32 ( column n = input
// channel n / 49, tap n % 49; zeros beyond column 146 ), so that a wave instruction of the main kernel reads 1 KB on end.
// ( Read column by column, 256 bytes per lane, every instruction touched 64 cache lines, five times eight times a tile:
// the refills of the first-level cache from the second took longer than the products. )
__global__ __launch_bounds__( 256 ) void packStemFilterKernel( const float* filter, float* packed )
{
	const int idx = blockIdx.x * 256 + threadIdx.x;
	if( idx >= SgPackedFilterFloats ) {
		return;
	}
	const int e = idx & 3, lane = ( idx >> 2 ) & 63, i = ( idx >> 8 ) & 7, chunk = idx >> 11;
	const int n = chunk * 32 + ( lane & 31 ), k = 32 * ( lane >> 5 ) + 4 * i + e;
	packed[idx] = n < SgColumns ? filter[k * SgColumns + ( n % 49 ) * 3 + n / 49] : 0.f;
}

__global__ __launch_bounds__( 256, 2 )
void stemInputGradientKernel( const float* outputDiff, const float* columns, float* tileWindows,
	int outH, int outW, int tilesY, int tilesX, int totalTiles )
{
	// ( + a place per lane for the columns of padding, + a word that stays zero )
	__shared__ __attribute__( ( aligned( 16 ) ) ) float windows[4][SgWaveFloats + 64 + 4];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
	// ( a row of pixels passes through the wave's window before the window is cleared for the tile )
	static_assert( 16 * SgStagePitch <= SgWaveFloats, "the staging row fits the window" );
	float* const stage = windows[wave];
	// operand row rho of block b: pixel x = 4 ( 2 * bit 2 of rho + bit 3 of rho ) + ( rho & 3 ), y = 4 ( 2 b + bit 4 of rho ) + wave;
	// as accumulator row rho = 8 q + 4 half + i that is X = 2 half + ( q & 1 ), band 2 b + ( q >> 1 )
	const int ownX = 4 * ( 2 * ( ( l32 >> 2 ) & 1 ) + ( ( l32 >> 3 ) & 1 ) ) + ( l32 & 3 );
	int rowTerm[2][4];
#pragma unroll
	for( int b = 0; b < 2; ++b ) {
#pragma unroll
		for( int q = 0; q < 4; ++q ) {
			const int x4 = 4 * ( 2 * half + ( q & 1 ) );
			const int band = 2 * b + ( q >> 1 );
			rowTerm[b][q] = band * SgBandFloats + 2 * x4 * 3;
		}
	}
	int columnTerm[5];
#pragma unroll
	for( int chunk = 0; chunk < 5; ++chunk ) {
		const int n = chunk * 32 + l32;
		const int c = n / 49, tap = n - c * 49, ky = tap / 7, kx = tap - ky * 7;
		columnTerm[chunk] = n < SgColumns ? ( ky * SgWindow + kx ) * 3 + c : 0;
	}
	const bool paddingColumn = 4 * 32 + l32 >= SgColumns; // ( in the last chunk )
	const __amdgpu_buffer_rsrc_t source = makeBuffer( outputDiff );
	// the filter as the lanes want it: [chunk][i][lane][4], see packStemFilterKernel
	const __amdgpu_buffer_rsrc_t filterColumns = __builtin_amdgcn_make_buffer_rsrc( const_cast<float*>( columns ), 0, SgPackedFilterFloats * 4, 0x00020000 );
	float* const window = windows[wave];
	if( lane == 0 ) {
		window[SgWaveFloats + 64] = 0.f;
	}
	// The wave's four rows of 16 pixels ( 4 KB each, contiguous ) are fetched as they lie, a wave instruction 1 KB on end,
	// and turned into the operand's layout ( a lane: 32 values of one pixel ) through LDS. Fetched in that layout
	// directly, every instruction touched 64 cache lines for 16 bytes each and came back for them seven more times
	// after the other waves' fetches had pushed them out.
	float4 fetched[4][4];
	auto request = [&]( int t ) {
		const int tx = t % tilesX;
		const int ty = ( t / tilesX ) % tilesY;
		const int n = t / ( tilesX * tilesY );
#pragma unroll
		for( int band = 0; band < 4; ++band ) {
			const int sy = 16 * ty + 4 * band + wave;
#pragma unroll
			for( int m = 0; m < 4; ++m ) {
				const int sx = 16 * tx + 4 * m + ( lane >> 4 );
				const unsigned at = ( t < totalTiles && sy < outH && sx < outW )
					? static_cast<unsigned>( ( ( n * outH + sy ) * outW + sx ) * 64 + ( lane & 15 ) * 4 ) * 4u : OutOfRange;
				fetched[band][m] = bufferLoad4( source, at );
			}
		}
	};
	for( int t = blockIdx.x; t < totalTiles; t += gridDim.x ) {
		request( t );
		float4 a[2][8];
#pragma unroll
		for( int band = 0; band < 4; ++band ) {
#pragma unroll
			for( int m = 0; m < 4; ++m ) {
				*reinterpret_cast<float4*>( stage + ( 4 * m + ( lane >> 4 ) ) * SgStagePitch + ( lane & 15 ) * 4 ) = fetched[band][m];
			}
			__builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
			__builtin_amdgcn_wave_barrier();
			__builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );
			if( ( l32 >> 4 ) == ( band & 1 ) ) {
#pragma unroll
				for( int i = 0; i < 8; ++i ) {
					a[band >> 1][i] = *reinterpret_cast<const float4*>( stage + ownX * SgStagePitch + 32 * half + 4 * i );
				}
			}
			__builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
			__builtin_amdgcn_wave_barrier();
			__builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );
		}
		float4 w[8];
#pragma unroll
		for( int i = 0; i < 8; ++i ) {
			w[i] = bufferLoad4( filterColumns, i * 1024u + lane * 16u );
		}
		// ( nobody reads this wave's window of the tile before any more: the barrier at the end of the tile )
		for( int i = lane; i < SgWaveFloats; i += 64 ) {
			window[i] = 0.f;
		}
#pragma unroll
		for( int chunk = 0; chunk < 5; ++chunk ) {
			stemAcc acc[2];
#pragma unroll
			for( int b = 0; b < 2; ++b ) {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					acc[b][r] = 0.f;
				}
			}
#pragma unroll
			for( int i = 0; i < 8; ++i ) {
				acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[0][i].x, w[i].x, acc[0], 0, 0, 0 );
				acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[1][i].x, w[i].x, acc[1], 0, 0, 0 );
				acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[0][i].y, w[i].y, acc[0], 0, 0, 0 );
				acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[1][i].y, w[i].y, acc[1], 0, 0, 0 );
				acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[0][i].z, w[i].z, acc[0], 0, 0, 0 );
				acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[1][i].z, w[i].z, acc[1], 0, 0, 0 );
				acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[0][i].w, w[i].w, acc[0], 0, 0, 0 );
				acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32( a[1][i].w, w[i].w, acc[1], 0, 0, 0 );
			}
			if( chunk < 4 ) {
				// the next chunk's columns arrive while this chunk's products are added up
#pragma unroll
				for( int i = 0; i < 8; ++i ) {
					w[i] = bufferLoad4( filterColumns, ( ( chunk + 1 ) * 8 + i ) * 1024u + lane * 16u );
				}
			}
#pragma unroll
			for( int i = 0; i < 4; ++i ) {
				float before[2][4];
				// ( columns of padding hold zeros; they go to a place of the lane's own )
				const int columnPart = ( chunk == 4 && paddingColumn ) ? -1 : columnTerm[chunk] + 6 * i;
#pragma unroll
				for( int b = 0; b < 2; ++b ) {
#pragma unroll
					for( int q = 0; q < 4; ++q ) {
						before[b][q] = window[columnPart < 0 ? SgWaveFloats + lane : rowTerm[b][q] + columnPart];
					}
				}
#pragma unroll
				for( int b = 0; b < 2; ++b ) {
#pragma unroll
					for( int q = 0; q < 4; ++q ) {
						window[columnPart < 0 ? SgWaveFloats + lane : rowTerm[b][q] + columnPart] = before[b][q] + acc[b][q * 4 + i];
					}
				}
				__builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
				__builtin_amdgcn_wave_barrier();
				__builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );
			}
		}
		__syncthreads();
		// row wy of the tile's window: from wave w the band with 0 <= wy - 8 band - 2 w <= 6, if there is one
		float* const out = tileWindows + static_cast<long long>( t ) * SgWindowFloats;
		// ( half a workgroup per row, a thread per value of the row: which bands a row takes is the same for the whole
		// half, so the addresses come from the scalar unit; what a wave has no band for is read from a word that holds
		// zero, so that all the reads of a thread can be in flight together )
		{
			const int column = threadIdx.x & 127;
			if( column < SgWindow * 3 ) {
				float sums[( SgWindow + 1 ) / 2];
#pragma unroll
				for( int step = 0; step < ( SgWindow + 1 ) / 2; ++step ) {
					const int wy = __builtin_amdgcn_readfirstlane( 2 * step + ( static_cast<int>( threadIdx.x ) >> 7 ) );
					sums[step] = 0.f;
#pragma unroll
					for( int w4 = 0; w4 < 4; ++w4 ) {
						const int band = ( wy - 2 * w4 ) >> 3; // ( floor: negative for wy < 2 w )
						const int ky = wy - 2 * w4 - 8 * band;
						const bool has = band >= 0 && band < 4 && ky <= 6 && wy < SgWindow;
						sums[step] += windows[w4][has ? band * SgBandFloats + ky * ( SgWindow * 3 ) + column : SgWaveFloats + 64];
					}
				}
#pragma unroll
				for( int step = 0; step < ( SgWindow + 1 ) / 2; ++step ) {
					const int wy = __builtin_amdgcn_readfirstlane( 2 * step + ( static_cast<int>( threadIdx.x ) >> 7 ) );
					if( wy < SgWindow ) {
						out[wy * ( SgWindow * 3 ) + column] = sums[step];
					}
				}
			}
		}
		__syncthreads();
	}
}

// input pixel ( gy, gx ): window row gy + 3 - 32 ty of tile row ty, for the one or two ty that have such a row
// ( a row of workgroups per SgGatherRows rows of the batch's images: what depends on the row is scalar arithmetic, and a
// thread has several rows' reads in flight )
constexpr int SgGatherRows = 8;

__global__ __launch_bounds__( 256 )
void stemGatherWindowsKernel( const float* tileWindows, const float* freeTerm, float* inputDiff, int height, int width,
	int tilesY, int tilesX, int rows )
{
	const int j = blockIdx.x * 256 + threadIdx.x;
	if( j >= width * 3 ) {
		return;
	}
	const int gx = j / 3, c = j - gx * 3;
	const float bias = freeTerm != nullptr ? freeTerm[c] : 0.f;
	const int tx1 = ( gx + 3 ) >> 5;
	const int wx1 = gx + 3 - 32 * tx1, wx0 = wx1 + 32; // in tile tx1 and in the one to its left
	const bool has1 = tx1 < tilesX, has0 = tx1 >= 1 && wx0 < SgWindow;
	float sums[SgGatherRows];
#pragma unroll
	for( int r = 0; r < SgGatherRows; ++r ) {
		const int row = blockIdx.y * SgGatherRows + r;
		sums[r] = bias;
		if( row < rows ) {
			const int gy = row % height, n = row / height;
			const int ty1 = ( gy + 3 ) >> 5;
#pragma unroll
			for( int dy = 1; dy >= 0; --dy ) {
				const int ty = ty1 - dy, wy = gy + 3 - 32 * ty;
				if( ty >= 0 && ty < tilesY && wy < SgWindow ) {
					const float* const from = tileWindows + static_cast<long long>( ( n * tilesY + ty ) * tilesX ) * SgWindowFloats
						+ wy * ( SgWindow * 3 ) + c;
					if( has0 ) {
						sums[r] += from[( tx1 - 1 ) * SgWindowFloats + wx0 * 3];
					}
					if( has1 ) {
						sums[r] += from[tx1 * SgWindowFloats + wx1 * 3];
					}
				}
			}
		}
	}
#pragma unroll
	for( int r = 0; r < SgGatherRows; ++r ) {
		const int row = blockIdx.y * SgGatherRows + r;
		if( row < rows ) {
			inputDiff[static_cast<long long>( row ) * ( width * 3 ) + j] = sums[r];
		}
	}
}

// tiles of 16 x 16 output-gradient pixels, or 0 where the window-summing path does not apply
static long long stemInputGradientTiles( const nhConvDesc& d )
{
	if( d.filterHeight != 7 || d.filterWidth != 7 || d.strideHeight != 2 || d.strideWidth != 2 || d.dilationHeight != 1 || d.dilationWidth != 1
		|| d.paddingHeight != 3 || d.paddingWidth != 3 || d.channels != 3 || d.filterCount != 64 )
	{
		return 0;
	}
	const long long tiles = static_cast<long long>( d.batch ) * ceilDiv( d.resultHeight, 16 ) * ceilDiv( d.resultWidth, 16 );
	// ( a handful of tiles: the general path spreads further; rows of the batch are a grid dimension of the second launch )
	return tiles >= 32 && tiles * SgWindowFloats <= 0x7fffffffLL && static_cast<long long>( d.batch ) * d.height <= 65535LL * SgGatherRows ? tiles : 0;
}

static bool stemInputGradient( hipStream_t stream, const nhConvDesc& d, const float* outputDiff, const float* filter,
	const float* freeTerm, float* inputDiff, float* workspace )
{
	const long long tiles = stemInputGradientTiles( d );
	if( tiles == 0 || !isAligned16( outputDiff ) || !isAligned16( workspace )
		|| !fitsBuffer( 1, 0, static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth * 64 ) )
	{
		return false;
	}
	const int tilesY = ceilDiv( d.resultHeight, 16 ), tilesX = ceilDiv( d.resultWidth, 16 );
	// workspace: the filter in the main kernel's order, then every tile's window
	float* const columns = workspace;
	float* const tileWindows = workspace + SgPackedFilterFloats;
	hipLaunchKernelGGL( packStemFilterKernel, dim3( SgPackedFilterFloats / 256 ), dim3( 256 ), 0, stream, filter, columns );
	// two workgroups per compute unit that stay for their share of the tiles ( 228 us against 237 with a workgroup per tile;
	// letting half of them begin half a tile later, so that the two of a unit are in different phases, changed nothing )
	const unsigned groups = static_cast<unsigned>( tiles < 512 ? tiles : 512 );
	hipLaunchKernelGGL( stemInputGradientKernel, dim3( groups ), dim3( 256 ), 0, stream, outputDiff, columns, tileWindows,
		d.resultHeight, d.resultWidth, tilesY, tilesX, static_cast<int>( tiles ) );
	hipLaunchKernelGGL( stemGatherWindowsKernel, dim3( ceilDiv( d.width * 3, 256 ), ceilDiv( d.batch * d.height, SgGatherRows ) ), dim3( 256 ), 0, stream,
		tileWindows, freeTerm, inputDiff, d.height, d.width, tilesY, tilesX, d.batch * d.height );
	return true;
}

int convBackwardData( hipStream_t stream, const nhConvDesc& d, const float* outputDiff, const float* filter,
	const float* freeTerm, float* inputDiff, float* swappedFilter )
{
	if( static_cast<long long>( d.batch ) * d.height * d.width == 0 || d.channels == 0 ) {
		return NH_OK;
	}
	int rc = NH_OK;
	if( stemInputGradient( stream, d, outputDiff, filter, freeTerm, inputDiff, swappedFilter ) ) {
		return hipGetLastError() == hipSuccess ? NH_OK : NH_ERR_HIP;
	}
	if( convBackwardDataByClasses( stream, d, outputDiff, filter, freeTerm, inputDiff, swappedFilter, rc ) ) {
		return rc;
	}
	const int taps = d.filterHeight * d.filterWidth;
	const int filterSize = d.filterCount * taps * d.channels;
	hipLaunchKernelGGL( swapFilterChannelsKernel, dim3( ceilDiv( filterSize, 1024 ) ), dim3( 256 ), 0, stream,
		filter, swappedFilter, d.filterCount, taps, d.channels );
	CMatMulArgs args = {};
	args.A = outputDiff; args.B = swappedFilter; args.C = inputDiff; args.Bias = freeTerm;
	const long long m = static_cast<long long>( d.batch ) * d.height * d.width;
	args.M = static_cast<int>( m );
	args.N = d.channels;
	args.K = taps * d.filterCount;
	args.Lda = 0; args.Ldb = args.K; args.Ldc = d.channels;
	args.H = d.resultHeight; args.W = d.resultWidth; args.Cin = d.filterCount;
	args.Ho = d.height; args.Wo = d.width; args.Fh = d.filterHeight; args.Fw = d.filterWidth;
	args.PadH = -d.paddingHeight; args.PadW = -d.paddingWidth;
	args.StrideH = 1; args.StrideW = 1;
	args.DilH = -d.dilationHeight; args.DilW = -d.dilationWidth;
	args.UpH = d.strideHeight; args.UpW = d.strideWidth;
	if( args.M == 0 || args.N == 0 ) {
		return NH_OK;
	}
	const bool vec = isAligned16( outputDiff ) && isAligned16( swappedFilter ) && d.filterCount % 4 == 0
		&& fitsBuffer( 1, 0, static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth * d.filterCount )
		&& fitsBuffer( d.channels, args.K, args.K );
	if( vec && d.filterCount % NH_KSTEP == 0 && d.strideHeight == 1 && d.strideWidth == 1 ) {
		return launchMatMul<AM_ConvTaps, BM_RowsK>( stream, args, 1, true );
	}
	return launchMatMul<AM_Conv, BM_RowsK>( stream, args, 1, vec );
}

// filterDiff[co][kh,kw,ci] += sum over output pixels of outputDiff[pixel][co] * im2col( input )[pixel][kh,kw,ci]
int convLearnAdd( hipStream_t stream, const nhConvDesc& d, const float* input, const float* outputDiff, float* filterDiff )
{
	CMatMulArgs args = {};
	args.A = outputDiff; args.B = input; args.C = filterDiff;
	const long long pixels = static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth;
	args.M = d.filterCount;
	args.N = d.filterHeight * d.filterWidth * d.channels;
	args.K = static_cast<int>( pixels );
	args.Lda = d.filterCount; args.Ldb = 0; args.Ldc = args.N;
	args.H = d.height; args.W = d.width; args.Cin = d.channels;
	args.Ho = d.resultHeight; args.Wo = d.resultWidth; args.Fh = d.filterHeight; args.Fw = d.filterWidth;
	args.PadH = d.paddingHeight; args.PadW = d.paddingWidth;
	args.StrideH = d.strideHeight; args.StrideW = d.strideWidth;
	args.DilH = d.dilationHeight; args.DilW = d.dilationWidth;
	args.Accumulate = 1;
	args.ManySlices = 1;
	if( args.M == 0 || args.N == 0 || args.K == 0 ) {
		return NH_OK;
	}
	const bool fits = isAligned16( outputDiff ) && d.filterCount % 4 == 0
		&& fitsBuffer( pixels, d.filterCount, d.filterCount )
		&& fitsBuffer( 1, 0, static_cast<long long>( d.batch ) * d.height * d.width * d.channels );
	bool vec = fits && isAligned16( input ) && d.channels % 4 == 0;
	if( fits && d.channels % 4 != 0 && d.dilationWidth == 1 ) {
		// grey and RGB inputs: the columns walk each filter row's run of Fw * Cin image values, padded to a multiple of 4
		args.RowK = d.filterWidth * d.channels;
		args.RowPitch = ( args.RowK + 3 ) / 4 * 4;
		args.BFloats = d.batch * d.height * d.width * d.channels;
		args.N = d.filterHeight * args.RowPitch; // Ldc keeps the filter's own row length
		vec = true;
	}
	return launchMatMul<AM_RowsM, BM_ConvN>( stream, args, 1, vec );
}

} // namespace nh

// ---------------------------------------------------------------------------------------------------------
// C ABI

using namespace nh;

extern "C" {

int nhMultiplyMatrixByTransposedMatrix( nhStream s, const float* first, int firstHeight, int firstWidth,
	int firstRowSize, const float* second, int secondHeight, int secondRowSize,
	float* result, int resultRowSize, int resultBufferSize )
{
	NH_REQUIRE( firstHeight >= 0 && firstWidth >= 0 && secondHeight >= 0 );
	NH_REQUIRE( firstRowSize >= firstWidth && secondRowSize >= firstWidth && resultRowSize >= secondHeight );
	// resultBufferSize is not looked at: the reference CPU engine ignores it (src/CPU/CpuMathEngineBlas.cpp:906-918)
	// and CFullyConnectedLayer::RunOnce passes 0 (NeoML/src/Dnn/Layers/FullyConnectedLayer.cpp:91-94)
	( void )resultBufferSize;
	// ( on a stream that puts small calls aside the product waits for the call behind it: a free term added to its rows
	// goes into the same launch )
	if( deferProduct( s, first, firstRowSize, second, secondRowSize, result, resultRowSize, firstHeight, secondHeight, firstWidth ) ) {
		return NH_OK;
	}
	return matMulNT( toStream( s ), first, firstRowSize, second, secondRowSize, result, resultRowSize,
		firstHeight, secondHeight, firstWidth, 1, 0, 0, 0, nullptr, false );
}

int nhBatchMultiplyMatrixByTransposedMatrix( nhStream s, int batchSize, const float* first, int firstHeight,
	int firstWidth, const float* second, int secondHeight, float* result, int resultBufferSize )
{
	NH_REQUIRE( batchSize >= 0 && firstHeight >= 0 && firstWidth >= 0 && secondHeight >= 0 );
	NH_REQUIRE( static_cast<long long>( batchSize ) * firstHeight * secondHeight <= resultBufferSize );
	return matMulNT( toStream( s ), first, firstWidth, second, firstWidth, result, secondHeight,
		firstHeight, secondHeight, firstWidth, batchSize,
		static_cast<long long>( firstHeight ) * firstWidth, static_cast<long long>( secondHeight ) * firstWidth,
		static_cast<long long>( firstHeight ) * secondHeight, nullptr, false );
}

int nhBatchMultiplyMatrixByMatrix( nhStream s, int batchSize, const float* first, int firstHeight,
	int firstWidth, const float* second, int secondWidth, float* result, int resultBufferSize )
{
	NH_REQUIRE( batchSize >= 0 && firstHeight >= 0 && firstWidth >= 0 && secondWidth >= 0 );
	NH_REQUIRE( static_cast<long long>( batchSize ) * firstHeight * secondWidth <= resultBufferSize );
	// ( on a stream that puts calls aside a batch of small products waits for the call behind it: CLinearLayer's multiplier
	// behind the QK^T of an attention layer becomes part of the launch )
	if( deferBatchedProduct( s, batchSize, first, firstHeight, firstWidth, second, secondWidth, result ) ) {
		return NH_OK;
	}
	return matMulNN( toStream( s ), first, firstWidth, second, secondWidth, result, secondWidth,
		firstHeight, secondWidth, firstWidth, batchSize,
		static_cast<long long>( firstHeight ) * firstWidth, static_cast<long long>( firstWidth ) * secondWidth,
		static_cast<long long>( firstHeight ) * secondWidth, false, nullptr, nullptr );
}

int nhMultiplyTransposedMatrixByMatrixAndAdd( nhStream s, const float* first, int firstHeight, int firstWidth,
	int firstRowSize, const float* second, int secondWidth, int secondRowSize,
	float* result, int resultRowSize, int resultBufferSize )
{
	NH_REQUIRE( firstHeight >= 0 && firstWidth >= 0 && secondWidth >= 0 );
	NH_REQUIRE( firstRowSize >= firstWidth && secondRowSize >= secondWidth && resultRowSize >= secondWidth );
	NH_REQUIRE( firstWidth == 0 || static_cast<long long>( firstWidth - 1 ) * resultRowSize + secondWidth <= resultBufferSize );
	return matMulTN( toStream( s ), first, firstRowSize, second, secondRowSize, result, resultRowSize,
		firstWidth, secondWidth, firstHeight, 1, 0, 0, 0, true );
}

int nhBatchMultiplyTransposedMatrixByMatrix( nhStream s, int batchSize, const float* first, int firstHeight,
	int firstWidth, const float* second, int secondWidth, float* result, int resultBufferSize )
{
	NH_REQUIRE( batchSize >= 0 && firstHeight >= 0 && firstWidth >= 0 && secondWidth >= 0 );
	NH_REQUIRE( static_cast<long long>( batchSize ) * firstWidth * secondWidth <= resultBufferSize );
	return matMulTN( toStream( s ), first, firstWidth, second, secondWidth, result, secondWidth,
		firstWidth, secondWidth, firstHeight, batchSize,
		static_cast<long long>( firstHeight ) * firstWidth, static_cast<long long>( firstHeight ) * secondWidth,
		static_cast<long long>( firstWidth ) * secondWidth, false );
}

int nhPointwiseConvolutionWithActivation( nhStream s, const float* source, int rows, int channels,
	const float* filter, const float* freeTerm, int filterCount, int activation, float param, float* result )
{
	NH_REQUIRE( source != nullptr && filter != nullptr && result != nullptr );
	NH_REQUIRE( rows >= 0 && channels > 0 && filterCount > 0 );
	const CFusedActivation act = { activation, param };
	return matMulNTFused( toStream( s ), source, channels, filter, channels, result, filterCount, rows, filterCount, channels,
		1, 0, 0, 0, freeTerm, false, act, nullptr );
}

int nhInitBlobConvolution( nhConvDesc* d )
{
	NH_REQUIRE( d != nullptr );
	NH_REQUIRE( d->batch >= 0 && d->height > 0 && d->width > 0 && d->channels > 0 );
	NH_REQUIRE( d->filterCount > 0 && d->filterHeight > 0 && d->filterWidth > 0 );
	NH_REQUIRE( d->paddingHeight >= 0 && d->paddingWidth >= 0 );
	NH_REQUIRE( d->strideHeight > 0 && d->strideWidth > 0 && d->dilationHeight > 0 && d->dilationWidth > 0 );
	const int spanH = ( d->filterHeight - 1 ) * d->dilationHeight + 1;
	const int spanW = ( d->filterWidth - 1 ) * d->dilationWidth + 1;
	NH_REQUIRE( d->height + 2 * d->paddingHeight >= spanH && d->width + 2 * d->paddingWidth >= spanW );
	d->resultHeight = ( d->height + 2 * d->paddingHeight - spanH ) / d->strideHeight + 1;
	d->resultWidth = ( d->width + 2 * d->paddingWidth - spanW ) / d->strideWidth + 1;
	const long long m = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth;
	NH_REQUIRE( m <= 0x7fffffffLL );
	NH_REQUIRE( static_cast<long long>( d->batch ) * d->height * d->width * d->channels <= 0x7fffffffLL );
	NH_REQUIRE( m * d->filterCount <= 0x7fffffffLL );
	return NH_OK;
}

// What every convolution entry point asks of a descriptor. The result sizes need not be the ones nhInitBlobConvolution
// computes for equal padding on both sides: fewer or more rows ( columns ) are taken as a different padding at the end,
// as long as the padding at the end stays within the larger of the padding at the beginning and the filter's span - 1.
// The kernels read whatever lies beyond the image as zeros wherever it is, so the padding at the end needs no field.
static int checkedConvDesc( const nhConvDesc* d )
{
	NH_REQUIRE( d != nullptr );
	NH_REQUIRE( d->batch >= 0 && d->height > 0 && d->width > 0 && d->channels > 0 );
	NH_REQUIRE( d->filterCount > 0 && d->filterHeight > 0 && d->filterWidth > 0 );
	NH_REQUIRE( d->paddingHeight >= 0 && d->paddingWidth >= 0 );
	NH_REQUIRE( d->strideHeight > 0 && d->strideWidth > 0 && d->dilationHeight > 0 && d->dilationWidth > 0 );
	const int spanH = ( d->filterHeight - 1 ) * d->dilationHeight + 1;
	const int spanW = ( d->filterWidth - 1 ) * d->dilationWidth + 1;
	const int endH = d->paddingHeight > spanH - 1 ? d->paddingHeight : spanH - 1;
	const int endW = d->paddingWidth > spanW - 1 ? d->paddingWidth : spanW - 1;
	NH_REQUIRE( d->resultHeight >= 1 && d->resultHeight <= ( d->height + d->paddingHeight + endH - spanH ) / d->strideHeight + 1 );
	NH_REQUIRE( d->resultWidth >= 1 && d->resultWidth <= ( d->width + d->paddingWidth + endW - spanW ) / d->strideWidth + 1 );
	const long long m = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth;
	NH_REQUIRE( m <= 0x7fffffffLL );
	NH_REQUIRE( static_cast<long long>( d->batch ) * d->height * d->width * d->channels <= 0x7fffffffLL );
	NH_REQUIRE( m * d->filterCount <= 0x7fffffffLL );
	return NH_OK;
}

int nhBlobConvolutionBackwardWorkspaceSize( const nhConvDesc* d, size_t* bytes )
{
	const int rc = checkedConvDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( bytes != nullptr );
	*bytes = static_cast<size_t>( d->filterCount ) * d->filterHeight * d->filterWidth * d->channels * sizeof( float );
	// ( the stem's input gradient: the filter with its columns padded, and the windows that its tiles leave there )
	const size_t stemTiles = static_cast<size_t>( stemInputGradientTiles( *d ) );
	if( stemTiles > 0 ) {
		*bytes = ( SgPackedFilterFloats + stemTiles * SgWindowFloats ) * sizeof( float );
	}
	return NH_OK;
}

int nhBlobConvolutionBackward( nhStream s, const nhConvDesc* d, const float* outputDiff, const float* filter,
	const float* freeTerm, float* inputDiff, void* workspace, size_t workspaceSize )
{
	size_t need = 0;
	const int rc = nhBlobConvolutionBackwardWorkspaceSize( d, &need );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( outputDiff != nullptr && filter != nullptr && inputDiff != nullptr );
	NH_REQUIRE( workspace != nullptr && workspaceSize >= need && isAligned16( workspace ) );
	NH_REQUIRE( static_cast<long long>( d->filterCount ) * d->filterHeight * d->filterWidth * d->channels <= 0x7fffffffLL );
	return convBackwardData( toStream( s ), *d, outputDiff, filter, freeTerm, inputDiff, static_cast<float*>( workspace ) );
}

int nhBlobConvolutionLearnAdd( nhStream s, const nhConvDesc* d, const float* input, const float* outputDiff, float* filterDiff )
{
	const int rc = checkedConvDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( input != nullptr && outputDiff != nullptr && filterDiff != nullptr );
	return convLearnAdd( toStream( s ), *d, input, outputDiff, filterDiff );
}

int nhBlobConvolution( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result )
{
	// ( on a stream that puts calls aside the convolution waits for the call behind it: a ReLU over its result in place
	// goes into the same launch )
	if( d != nullptr && source != nullptr && filter != nullptr && result != nullptr && checkedConvDesc( d ) == NH_OK
		&& deferConvolution( s, false, *d, source, filter, freeTerm, result ) )
	{
		return NH_OK;
	}
	return nhBlobConvolutionWithActivation( s, d, source, filter, freeTerm, NH_ACT_NONE, 0.f, result );
}

int nhBlobConvolutionNoAlloc( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result )
{
	NH_REQUIRE( d != nullptr && source != nullptr && filter != nullptr && result != nullptr );
	int rc = checkedConvDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	CSliceMeeting meeting = {};
	rc = noAllocMeeting( meeting );
	if( rc != NH_OK ) {
		return rc;
	}
	const CFusedActivation none = { NH_ACT_NONE, 0.f };
	return convImplicitGemm( toStream( s ), *d, source, filter, freeTerm, result, none, &meeting );
}

int nhStreamBindPool( nhStream s, nhPool pool )
{
	return bindSliceScratchPool( toStream( s ), pool );
}

int nhStreamReleaseScratch( nhStream s )
{
	NH_HIP( hipStreamSynchronize( toStream( s ) ) );
	releaseSliceScratch( toStream( s ), false );
	return NH_OK;
}

int nhBlobConvolutionWithActivation( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, int activation, float param, float* result )
{
	NH_REQUIRE( d != nullptr && source != nullptr && filter != nullptr && result != nullptr );
	const int rc = checkedConvDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	const CFusedActivation act = { activation, param };
	return convImplicitGemm( toStream( s ), *d, source, filter, freeTerm, result, act );
}

} // extern "C"
