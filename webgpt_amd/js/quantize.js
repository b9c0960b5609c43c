// Weight-only int8 quantisation of a linear weight: the host side of other/int8-gemm.js.
//
// quantizeMatrix is the reference's function of that name (other/int8-gemm.js:25-46) with the
// one change its own header asks for (line 4: a vector-wise absmax instead of a global one):
// the absmax is taken per output column of the row-major [rows, cols] matrix. The result is
// what the library's int8 entry points consume: words [rows, cols/4] with four consecutive
// columns per 32-bit word (element 0 in bits 0-7) and one fp32 scale per column.
// dequantizeMatrix is other/int8-gemm.js:48-62 with the column's absmax (float64 arithmetic,
// one rounding on the store into the Float32Array). The kernels compute
// float(q) / 127.0f * scale in fp32 as the shader does (int8-gemm.js:126-132), which can
// differ from it by one ulp.
"use strict";

function absmaxColumns(matrix, rows, cols) {
  const absmax = new Float64Array(cols);
  for (let k = 0; k < rows; k++) {
    const row = k * cols;
    for (let n = 0; n < cols; n++) absmax[n] = Math.max(absmax[n], Math.abs(matrix[row + n]));
  }
  return absmax;
}

// `absmax` (optional): a number (the reference's single global value) or one value per column.
function quantizeMatrix(matrix, rows, cols, absmax) {
  if (cols % 4 !== 0) throw new Error("Cols must be divisible by 4.");
  if (matrix.length !== rows * cols) throw new Error("quantizeMatrix: matrix does not hold rows * cols values.");
  const am = absmax === undefined ? absmaxColumns(matrix, rows, cols) : typeof absmax === "number" ? new Float64Array(cols).fill(absmax) : Float64Array.from(absmax);
  const quantizedMatrix = new Int32Array((rows * cols) / 4);
  const wordsPerRow = cols / 4;
  for (let k = 0; k < rows; k++) {
    for (let j = 0; j < wordsPerRow; j++) {
      const i = k * cols + 4 * j, n = 4 * j;
      quantizedMatrix[k * wordsPerRow + j] =
        (Math.round((matrix[i] / am[n]) * 127) & 0xff) |
        ((Math.round((matrix[i + 1] / am[n + 1]) * 127) & 0xff) << 8) |
        ((Math.round((matrix[i + 2] / am[n + 2]) * 127) & 0xff) << 16) |
        ((Math.round((matrix[i + 3] / am[n + 3]) * 127) & 0xff) << 24);
    }
  }
  return { quantizedMatrix, scale: Float32Array.from(am) };
}

function dequantizeMatrix(quantizedMatrix, scale, rows, cols) {
  const matrix = new Float32Array(rows * cols);
  const wordsPerRow = cols / 4;
  for (let k = 0; k < rows; k++) {
    for (let j = 0; j < wordsPerRow; j++) {
      const packedValue = quantizedMatrix[k * wordsPerRow + j];
      const i = k * cols + 4 * j, n = 4 * j;
      matrix[i] = (((packedValue << 24) >> 24) / 127.0) * scale[n];
      matrix[i + 1] = (((packedValue << 16) >> 24) / 127.0) * scale[n + 1];
      matrix[i + 2] = (((packedValue << 8) >> 24) / 127.0) * scale[n + 2];
      matrix[i + 3] = ((packedValue >> 24) / 127.0) * scale[n + 3];
    }
  }
  return matrix;
}

module.exports = { quantizeMatrix, dequantizeMatrix, absmaxColumns };
