// Input kernels for the front-end tests, written in the style of the TVM output the
// reference fuses: extern "C", three pointers, static __shared__ tiles, __syncthreads(),
// multi-dimensional grid and block indices.  (Plain C subset: compiles as HIP unchanged.)

// C[128,128] = A[128,64] . B[64,128]; block (16,16,1), grid (8,8,1), 16x16 tiles of A and B in LDS
extern "C" __global__ void __launch_bounds__(256) mm_tiled(float* __restrict__ A, float* __restrict__ B, float* __restrict__ C) {
  __shared__ float A_shared[256];
  __shared__ float B_shared[256];
  float acc = 0.000000e+00f;
  for (int k_outer = 0; k_outer < 4; ++k_outer) {
    __syncthreads();
    A_shared[((((int)threadIdx.y) * 16) + ((int)threadIdx.x))] = A[((((((int)blockIdx.y) * 1024) + (((int)threadIdx.y) * 64)) + (k_outer * 16)) + ((int)threadIdx.x))];
    B_shared[((((int)threadIdx.y) * 16) + ((int)threadIdx.x))] = B[((((k_outer * 2048) + (((int)threadIdx.y) * 128)) + (((int)blockIdx.x) * 16)) + ((int)threadIdx.x))];
    __syncthreads();
    for (int k_inner = 0; k_inner < 16; ++k_inner) {
      acc = (acc + (A_shared[((((int)threadIdx.y) * 16) + k_inner)] * B_shared[((k_inner * 16) + ((int)threadIdx.x))]));
    }
  }
  C[((((((int)blockIdx.y) * 2048) + (((int)threadIdx.y) * 128)) + (((int)blockIdx.x) * 16)) + ((int)threadIdx.x))] = acc;
}

// Y[r, c] = X[r, c] * S[r] + S[(r + 1) % 128] for X[128, 256]; block (64,1,2), grid (4,16,1):
// a block owns 8 rows x 64 columns (4 rows per threadIdx.z), the 9 scales it needs go through LDS
extern "C" __global__ void __launch_bounds__(128) row_scale(float* __restrict__ X, float* __restrict__ S, float* __restrict__ Y) {
  __shared__ float S_shared[9];
  if (((((int)threadIdx.z) * 64) + ((int)threadIdx.x)) < 9) {
    S_shared[((((int)threadIdx.z) * 64) + ((int)threadIdx.x))] = S[((((((int)blockIdx.y) * 8) + (((int)threadIdx.z) * 64)) + ((int)threadIdx.x)) % 128)];
  }
  __syncthreads();
  for (int r = 0; r < 4; ++r) {
    Y[((((((int)blockIdx.y) * 2048) + (((int)threadIdx.z) * 1024)) + (r * 256)) + ((((int)blockIdx.x) * 64) + ((int)threadIdx.x)))] = ((X[((((((int)blockIdx.y) * 2048) + (((int)threadIdx.z) * 1024)) + (r * 256)) + ((((int)blockIdx.x) * 64) + ((int)threadIdx.x)))] * S_shared[((((int)threadIdx.z) * 4) + r)]) + S_shared[(((((int)threadIdx.z) * 4) + r) + 1)]);
  }
}

// Z[i] = P[i] > Q[i] ? P[i] : Q[i] over 10240 floats; 152-thread blocks (not a multiple of 64), grid (68,1,1), no LDS
extern "C" __global__ void __launch_bounds__(152) ew_max(float* __restrict__ P, float* __restrict__ Q, float* __restrict__ Z) {
  if (((((int)blockIdx.x) * 152) + ((int)threadIdx.x)) < 10240) {
    Z[((((int)blockIdx.x) * 152) + ((int)threadIdx.x))] = ((P[((((int)blockIdx.x) * 152) + ((int)threadIdx.x))] > Q[((((int)blockIdx.x) * 152) + ((int)threadIdx.x))]) ? P[((((int)blockIdx.x) * 152) + ((int)threadIdx.x))] : Q[((((int)blockIdx.x) * 152) + ((int)threadIdx.x))]);
  }
}
