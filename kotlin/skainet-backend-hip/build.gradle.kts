// skainet-backends/skainet-backend-hip: the kernel SPI on an MI355X through libskainet_hip.so (Panama FFM, JVM only).
// Add `include(":skainet-backends:skainet-backend-hip")` to settings.gradle.kts; nothing else in the build changes.
plugins {
    alias(libs.plugins.kotlinMultiplatform)
    alias(libs.plugins.vanniktech.mavenPublish)
}

kotlin {
    explicitApi()
    jvm()
    jvmToolchain(22)                      // java.lang.foreign is final from 22 on

    sourceSets {
        val jvmMain by getting {
            dependencies {
                api(project(":skainet-backends:skainet-backend-api"))
                implementation(project(":skainet-lang:skainet-lang-core"))
            }
        }
        val jvmTest by getting {
            dependencies {
                implementation(kotlin("test"))
            }
        }
    }
}

// libskainet_hip.so is found through java.library.path / LD_LIBRARY_PATH (System.mapLibraryName("skainet_hip")); a
// machine without it, or without a gfx950 device, leaves the provider unavailable and the CPU tiers in charge.
tasks.withType<Test>().configureEach {
    jvmArgs("--enable-native-access=ALL-UNNAMED")
    systemProperty("java.library.path", (findProperty("skainetHipLibDir") as String?) ?: "")
}
