'use strict';
/** Shared by the CPU and GPU tiers: a weight shard with string and complex64 entries, and its check. */
module.exports = (tf, h) => {
// The byte layout that the reference's encodeWeights tests assert for string and complex64 tensors
// (tfjs-core/src/io/io_utils_test.ts:331-425: every string element a little-endian uint32 byte count
// and its UTF-8 bytes; complex64 as interleaved float32 pairs), decoded the way its decode test expects
// (io_utils_test.ts:503-528): each tensor comes back with the values that were encoded.
function referenceStringAndComplexShard() {
  const strings = [['a', 'bc', 'def', 'g'], [''], ['здраво', 'поздрав'], ['正常'], ['hello']];
  const specs = [
    {name: 'x1', dtype: 'string', shape: [2, 2]}, {name: 'x2', dtype: 'string', shape: []},
    {name: 'x3', dtype: 'string', shape: [2]}, {name: 'x4', dtype: 'string', shape: []},
    {name: 'x5', dtype: 'string', shape: []}, {name: 'i', dtype: 'int32', shape: [2, 2]},
    {name: 'c1', dtype: 'complex64', shape: [2]}, {name: 'c2', dtype: 'complex64', shape: []},
    {name: 'c3', dtype: 'complex64', shape: [1, 1]}
  ];
  const parts = [];
  strings.forEach(group => group.forEach(text => {
    const utf8 = Buffer.from(text, 'utf8');
    const count = Buffer.alloc(4);
    count.writeUInt32LE(utf8.length, 0);
    parts.push(count, utf8);
  }));
  parts.push(Buffer.from(new Int32Array([10, 20, 30, 40]).buffer));
  parts.push(Buffer.from(new Float32Array([1, 1, 2, 2, 1, 2, 1, 2]).buffer));   // complex([1,2],[1,2]), 1+2i, [[1+2i]]
  const shard = Buffer.concat(parts);
  // the sizes the reference's test works out: 7 + 4*4, 4, 13*2 + 2*4, 6 + 4, 5 + 4 bytes of strings
  h.assertEqual(shard.length, (7 + 16) + 4 + (26 + 8) + (6 + 4) + (5 + 4) + 16 + 32);
  h.assertEqual(shard.readUInt32LE(27), 12);   // 'здраво' starts at byte 27 with a count of 12 (io_utils_test.ts:397-398)
  return {shard: new Uint8Array(shard).buffer, specs, strings};
}

function checkStringAndComplexWeights(out, strings) {
  const text = t => Array.from(t.dataSync()).map(b => Buffer.from(b).toString('utf8'));
  ['x1', 'x2', 'x3', 'x4', 'x5'].forEach((name, k) => {
    h.assertEqual(out[name].dtype, 'string');
    h.assertEqual(text(out[name]), strings[k]);
  });
  h.assertEqual(out.x1.shape, [2, 2]);
  h.assertEqual(Array.from(out.i.dataSync()), [10, 20, 30, 40]);
  h.assertEqual(out.c1.dtype, 'complex64');
  h.assertEqual(Array.from(out.c1.dataSync()), [1, 1, 2, 2]);
  h.assertEqual(Array.from(out.c2.dataSync()), [1, 2]);
  h.assertEqual(out.c3.shape, [1, 1]);
  h.assertEqual(Array.from(tf.real(out.c1).dataSync()), [1, 2]);
  h.assertEqual(Array.from(tf.imag(out.c3).dataSync()), [2]);
}

  return {referenceStringAndComplexShard, checkStringAndComplexWeights};
};
