/* TEST INFRASTRUCTURE ONLY (checker for tests/, smoke and the cpu_baseline leg of the bench).
 *
 * The 126 ascending positive fp32 magnitudes of the dynamic 8-bit float codebook, as IEEE-754
 * binary32 bit patterns.  Source of the values: the dataset "/Default" (126x1 fp32) of the
 * reference's data file source/8bit_floats.hdf5 (raw little-endian payload at byte offset
 * 2144..2647), which the reference uploads once in ClusterNet::init (source/clusterNet.cpp:73,
 * loader source/util.cu:100-131).  The bits carry fp32 rounding noise, so they are data, not a
 * formula.  SHA-256 of the 504 payload bytes:
 *   c2dbfffe982a2fc5430f56cbb44857fe8e6b610b4445f3dae2a64b0b6c977a37
 */
#ifndef CN_ORACLE_TABLE_8BIT_H
#define CN_ORACLE_TABLE_8BIT_H
#include <stdint.h>

static const uint32_t cn_oracle_table_bits[126] = {
    0x36388ca4u, 0x36f34506u, 0x379d4952u, 0x38180b24u, 0x38766a54u, 0x38b4e11du,
    0x3916bb99u, 0x39727bb3u, 0x39a71de7u, 0x39d4fdf4u, 0x3a07fcb9u, 0x3a2c0831u,
    0x3a5013a8u, 0x3a741f20u, 0x3a9fbe77u, 0x3ad91687u, 0x3b09374cu, 0x3b25e354u,
    0x3b428f5cu, 0x3b5f3b64u, 0x3b7be76du, 0x3b8c49bau, 0x3b9eb852u, 0x3bb53f7du,
    0x3bcbc6a7u, 0x3be24dd2u, 0x3bf8d4fdu, 0x3c07ae14u, 0x3c12f1a9u, 0x3c1e353eu,
    0x3c35c28fu, 0x3c59999au, 0x3c7d70a4u, 0x3c90a3d7u, 0x3ca28f5cu, 0x3cb47ae1u,
    0x3cc66666u, 0x3cd851ecu, 0x3cea3d71u, 0x3cfc28f6u, 0x3d070a3du, 0x3d100000u,
    0x3d18f5c3u, 0x3d21eb85u, 0x3d2ae148u, 0x3d33d70au, 0x3d3f5c29u, 0x3d4d70a4u,
    0x3d5b851eu, 0x3d699999u, 0x3d77ae14u, 0x3d82e147u, 0x3d89eb85u, 0x3d90f5c2u,
    0x3d97ffffu, 0x3d9f0a3du, 0x3da6147au, 0x3dad1eb7u, 0x3db428f5u, 0x3dbb3332u,
    0x3dc23d6fu, 0x3dc947adu, 0x3dd80000u, 0x3dee6666u, 0x3e026666u, 0x3e0d999au,
    0x3e18cccdu, 0x3e240000u, 0x3e2f3333u, 0x3e3a6666u, 0x3e45999au, 0x3e50cccdu,
    0x3e5c0000u, 0x3e673333u, 0x3e726666u, 0x3e7d999au, 0x3e846666u, 0x3e8a0000u,
    0x3e8f999au, 0x3e953333u, 0x3e9acccdu, 0x3ea06666u, 0x3ea60000u, 0x3eab999au,
    0x3eb13333u, 0x3eb6cccdu, 0x3ebc6666u, 0x3ec20000u, 0x3ec7999au, 0x3ecd3333u,
    0x3ed2cccdu, 0x3ed86666u, 0x3ede0000u, 0x3ee3999au, 0x3eeacccdu, 0x3ef39999u,
    0x3efc6666u, 0x3f029999u, 0x3f070000u, 0x3f0b6666u, 0x3f0fccccu, 0x3f143333u,
    0x3f189999u, 0x3f1d0000u, 0x3f216666u, 0x3f25ccccu, 0x3f2a3333u, 0x3f2e9999u,
    0x3f32ffffu, 0x3f376666u, 0x3f3bccccu, 0x3f403332u, 0x3f449999u, 0x3f48ffffu,
    0x3f4d6665u, 0x3f51ccccu, 0x3f563332u, 0x3f5a9998u, 0x3f5effffu, 0x3f636665u,
    0x3f67cccbu, 0x3f6c3332u, 0x3f709998u, 0x3f74fffeu, 0x3f796665u, 0x3f7dcccbu,
};

#endif
