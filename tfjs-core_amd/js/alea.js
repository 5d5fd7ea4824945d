'use strict';
// Alea, Johannes Baagoe's generator, in the variant the seedrandom package (2.4.3, a dependency
// of the reference: package.json) ships as seedrandom.alea; restated from its published
// description.  Returns a function giving doubles in [0, 1).
function alea(seed) {
  let n = 0xefc8249d;
  const mash = data => {
    for (let i = 0; i < data.length; i++) {
      n += data.charCodeAt(i);
      let h = 0.02519603282416938 * n;
      n = h >>> 0;
      h -= n;
      h *= n;
      n = h >>> 0;
      h -= n;
      n += h * 0x100000000;  // 2^32
    }
    return (n >>> 0) * 2.3283064365386963e-10;  // 2^-32
  };
  let s0 = mash(' '), s1 = mash(' '), s2 = mash(' '), c = 1;
  s0 -= mash(seed);
  if (s0 < 0) s0 += 1;
  s1 -= mash(seed);
  if (s1 < 0) s1 += 1;
  s2 -= mash(seed);
  if (s2 < 0) s2 += 1;
  return () => {
    const t = 2091639 * s0 + c * 2.3283064365386963e-10;
    s0 = s1;
    s1 = s2;
    return s2 = t - (c = t | 0);
  };
}

module.exports = {alea};
