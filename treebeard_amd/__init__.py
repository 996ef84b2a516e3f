"""MI355X-native decision-forest inference behind Treebeard's runtime surface."""
